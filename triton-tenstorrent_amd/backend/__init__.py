"""Plugin surface: ``compiler.TTBackend`` and ``driver.TTDriver``.

The package is named by ``name.conf`` the way the reference names its own
(backend/name.conf:1); Triton discovers it through the ``triton.backends`` entry
point group, and :func:`triton_tenstorrent_amd.backend.driver.activate` installs
the driver when another (the stock HIP one) is already active.
"""

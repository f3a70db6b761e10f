"""MI355X-native (gfx950) implementation of the kernels the triton-tenstorrent
plugin runs, behind the plugin's own backend/driver surface.

Layout:
  backend/compiler.py, backend/driver.py  the plugin API (target registration,
                                          launcher, device interface)
  runtime.py     ctypes binding of libttamd_rt.so (C ABI in include/ttamd_rt.h)
  jit.py         `kernel[grid](*args, **constexprs)` front-end for the prebuilt
                 kernels when Triton's JIT is not in the loop
  kernels.py     the example kernels' names/signatures and their host wrappers
  csrc/          HIP kernels and the C++ host runtime
"""
__version__ = "0.1.0"

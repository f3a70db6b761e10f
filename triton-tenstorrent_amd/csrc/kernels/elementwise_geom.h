// Launch geometry shared by the elementwise kernels and their host launcher.
#pragma once

namespace ewgeom {
constexpr int kThreads = 64;   // one wavefront per workgroup
constexpr int kVec = 1;        // 16-byte vectors per lane and operand: the streaming kernels
// sin and cos: one vector per lane like the other streaming kernels, now that the library routine for huge
// arguments sits behind a branch (while the compiler evaluated it for every element, 330 instructions of it, a
// wavefront needed two vectors in flight to hide its own arithmetic: 3.0 TB/s with one, 6.45 with two, 6.30 with
// four; behind the branch: 6.74 with one, 6.44 with two, at N = 2^28, beside exp at 6.72)
#ifndef TTAMD_EW_TRIG_VEC
#define TTAMD_EW_TRIG_VEC 1
#endif
constexpr int kVecTrig = TTAMD_EW_TRIG_VEC;
} // namespace ewgeom

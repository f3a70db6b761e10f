// Launch geometry shared by the elementwise kernels and their host launcher.
#pragma once

namespace ewgeom {
constexpr int kThreads = 64;   // one wavefront per workgroup
constexpr int kVec = 1;        // 16-byte vectors per lane and operand: the streaming kernels
// sin and cos spend about 120 VALU instructions per vector: with one vector per lane a wavefront has too little in
// flight to cover the memory latency behind that arithmetic (3.0 TB/s at N = 2^28; two: 6.45, four: 6.30, eight: 6.25)
#ifndef TTAMD_EW_HEAVY_VEC
#define TTAMD_EW_HEAVY_VEC 2
#endif
constexpr int kVecHeavy = TTAMD_EW_HEAVY_VEC;
} // namespace ewgeom

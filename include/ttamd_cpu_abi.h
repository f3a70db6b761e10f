/* Host support for kernels built with the reference's cpu/ calling convention
 *
 *     void kernel(user args..., int32_t *launch_sz, int32_t *launch_id, int8_t *smem, void *barrier);
 *
 * (cpu/lib/TritonCPUToLLVM/FuncOpToLLVM.cpp:44-65, cpu/lib/TritonCPUToLLVM/Utility.h:14-19):
 *   launch_sz = { gridX, gridY, gridZ, blockX, blockY, blockZ }
 *   launch_id = { block_start, block_end, thread_id, 0, 0 }       (GPUOpToLLVM.cpp:16-22)
 *   smem      = the block's shared memory, 64-byte aligned          (FuncOpToLLVM.cpp:150-162, TargetInfo.h:10)
 *   barrier   = opaque; the kernel hands it to the external function `_cpu_barrier` at every
 *               gpu.barrier (GPUOpToLLVM.cpp:196-237), which the host has to supply.
 *
 * The reference leaves the host side of this convention to its runtime dependency (the knexus
 * `device.load_library / lib.get_kernel / schedule.run` calls of backend/driver.py:68-74, 114-170), which
 * is not part of its tree.  libttamd_cpuabi.so supplies the one native piece such a host needs, the
 * barrier; the launcher itself (argument marshalling, one [block_start, block_end) range per worker,
 * one host thread per (worker, thread_id)) is triton_tenstorrent_amd/cpu_abi.py.
 *
 * This library runs kernels that the CALLER compiled for the host.  It is not a fallback for the gfx950
 * kernels of libttamd_rt.so and shares no code with them.
 */
#ifndef TTAMD_CPU_ABI_H
#define TTAMD_CPU_ABI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* What a kernel's gpu.barrier calls: returns once all `workers` threads of the barrier have arrived.
 * Reusable; a barrier of one worker returns at once. */
void _cpu_barrier(void *barrier);

/* A barrier for `workers` threads (>= 1), zero-initialised as the kernels assume; NULL on failure. */
void *ttamd_cpu_barrier_create(int32_t workers);
void ttamd_cpu_barrier_destroy(void *barrier);

/* `bytes` of zeroed shared memory aligned to 64 bytes (a distinct non-NULL pointer for bytes == 0). */
void *ttamd_cpu_smem_alloc(uint64_t bytes);
void ttamd_cpu_smem_free(void *smem);

/* Blocks [*start, *end) of `blocks` that worker `worker` of `workers` runs: contiguous ranges in worker
 * order, the first blocks % workers of them one block longer (the split of SPMDOpToD2M.cpp:38-112). */
void ttamd_cpu_block_range(int32_t blocks, int32_t workers, int32_t worker, int32_t *start, int32_t *end);

#ifdef __cplusplus
}
#endif
#endif

/*
 * Timing and tuning entry points of libcrow_hip.so that are NOT part of the drop-in boundary: nothing in the reference engine
 * corresponds to them and the Rust shim does not bind them.  They serve this repository's benchmark (bench.py) and its tests:
 * loops of launches timed inside the library between two HIP events on the launch stream, and the launch geometry of the NVFP4
 * GEMV family with the split forced.  The product ABI is include/crow_hip.h.
 */
#ifndef CROW_HIP_BENCH_H
#define CROW_HIP_BENCH_H
#include "crow_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* crow_hip_launch_dims with the GEMV split forced: `s` column slices per 16-row strip (blocks that hand their partial sums over through
 * the workspace) and `w` waves per block and tensor; 0 = the library's choice.  Every GEMV kernel is correct for every split:
 * this is for tuning and for tests.  Other kernels ignore s and w. */
int crow_hip_launch_dims_split(const char* name, uint32_t rows, uint32_t k_dim, uint32_t z, uint32_t s, uint32_t w, crow_dims* out);

/* `iters` back-to-back launches of `f` on the current stream between two events, launch i taking
 * the argument set vals[(i % n_sets) * n_vals ...] (rotating weight copies keep the working set
 * larger than the 256 MB memory-side cache).  Returns the mean microseconds per launch. */
int crow_hip_time_launches(crow_fn_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, const uint64_t* vals,
                           uint32_t n_vals, uint32_t n_sets, uint32_t iters, float* us_per_launch);
/* the same for a SEQUENCE of n_kernels launches per iteration (e.g. router -> gate|up -> down): dims[k] and
 * n_vals[k] per kernel; argument set s of iteration i = vals + (i % n_sets) * sum(n_vals), kernels back to back
 * inside it.  Returns the mean microseconds per iteration (per sequence). */
int crow_hip_time_sequence(uint32_t n_kernels, const crow_fn_t* fns, const crow_dims* dims, const uint32_t* n_vals,
                           const uint64_t* vals, uint32_t n_sets, uint32_t iters, float* us_per_iteration);

/* What a PURE READ of `bytes` (a multiple of 2304) takes on this device with nothing else in the kernel: `iters` back-to-back
 * launches of (blocks x threads) between two events, launch i reading the device buffer bufs[i % n_bufs] (rotating copies, as
 * above).  pattern 0: the GEMVs' own access pattern - the same three non-temporal loads per lane and 2304-byte group, four groups
 * in flight per wave; pattern 1: the textbook stream - 16 contiguous bytes per lane and load, eight loads in flight per lane,
 * non-temporal; pattern 2: the same with plain loads.  The benchmark reports the best of them beside each kernel as the chip's
 * ceiling for that many bytes. */
int crow_hip_time_pure_read(const uint64_t* bufs, uint32_t n_bufs, size_t bytes, uint32_t blocks, uint32_t threads, uint32_t pattern,
                            uint32_t iters, float* us_per_launch);

/* `iters` back-to-back replays on `stream` between two events; mean microseconds per replay */
int crow_hip_time_graph(void* graph_exec, void* stream, uint32_t iters, float* us_per_replay);

#ifdef __cplusplus
}
#endif
#endif

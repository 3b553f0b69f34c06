// NVFP4 GEMV family for gfx950: y[m][row] = gs * sum_k W[row][k] * x[m][k], M <= 4 activation rows.
//
// Mapping.  One wavefront owns one 64-row tile: lane l computes row l.  All lanes of a wave walk
// the same columns, so the activation is wave-uniform and is read through scalar loads into
// SGPRs; the FMA takes it as its scalar operand and nothing is ever shuffled between lanes.
// Weights are read exactly once, as 16-byte-per-lane loads that cover 1024 contiguous bytes per
// instruction (layout.h).  E2M1 pairs decode with v_cvt_scalef32_pk_f32_fp4 (exact), UE4M3 scales
// with v_cvt_f32_fp8 (exact on canonical bytes).
//
// FP32 accumulation order (per output row and activation row), documented because it differs
// from the reference CPU path's 8-lane order (cpu_nvfp4.rs:22-31) and from its GPU kernel of
// record (kernels_p2.rs:304-347); all three are within the same gamma bound of the exact sum:
//   for each 16-value sub-block, in column order:
//       part = fma(w15, x15, ... fma(w1, x1, w0 * x0))        (w exact, 16 fused steps)
//       acc  = fma(part, ue4m3(scale), acc)
//   a row split over S blocks of W waves: unit u = slice * W + wave owns panels u, u + S W, ...;
//   a block adds its waves' `acc` values in wave order, then the blocks' sums are added in
//   slice order (slice 0 first)
//   y = acc * gs                                               (gs last, as kernels_p2.rs:367)
// The order depends only on (K, slices), never on M: row m of an M-row launch is bit-identical to
// a one-row launch with the same slicing (the verify contract of kernels_p2.rs:391-396).
//
// Launch geometry: grid (S, row_tiles, Z), block 64 * W.  blockIdx.y = row tile, blockIdx.x = column
// slice, blockIdx.z = token group / expert combo.  The W waves of a block and the S blocks of a row
// tile deal the tile's 256-column panels round-robin: unit u = slice * W + wave takes panels u,
// u + S W, ...  (the split is chosen so that a wave usually owns one or two panels and all of the
// launch's waves are resident at once: every load of the launch is then in flight from the start).
// Waves combine through LDS in wave order; blocks combine through the library workspace: every
// block stores its partial sums, bumps the tile's arrival counter, and the block that arrives
// last adds all partials in slice order and writes y - deterministic whatever the arrival order.
// With S = 1 the workspace is not touched.
#pragma once
#include "device_common.h"

namespace crow {

enum Epilogue { EPI_SCALE = 0, EPI_SILU_GU = 1 };

struct GemvArgs {
    const unsigned char* w[2];  // tiled tensors (w[1] only for EPI_SILU_GU: the `up` matrix)
    const float* gs[2];
    const void* x;       // [M][x_stride] f32 (or bf16 when XBF16)
    size_t x_stride;     // elements between activation rows
    float* y;            // [M][y_stride]
    size_t y_stride;
    int k_dim, rows, m;  // m <= MMAX of the instantiation
    int* argmax_out;     // not null: also write the greedy argmax of y row 0 (fused lm_head head)
};

// 16 consecutive activation values of row m, wave-uniform (scalar loads)
template <bool XBF16>
struct XChunk;
template <>
struct XChunk<false> {
    float v[16];
    __device__ __forceinline__ void load(const void* x, size_t off) {
        const float* p = (const float*)x + off;
#pragma unroll
        for (int j = 0; j < 16; j++) v[j] = p[j];
    }
};
template <>
struct XChunk<true> {
    unsigned v[8];  // bf16 pairs
    __device__ __forceinline__ void load(const void* x, size_t off) {
        const unsigned* p = (const unsigned*)((const unsigned short*)x + off);
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = p[j];
    }
};

// one 16-value sub-block: two code words (w0: values 0..7, w1: values 8..15).  The chain is split
// into its first link and the rest so that a caller can place other work between them.
template <bool XBF16>
__device__ __forceinline__ float dot_head(unsigned w0, const XChunk<XBF16>& x);
template <bool XBF16>
__device__ __forceinline__ float dot_tail(float part, unsigned w0, unsigned w1, const XChunk<XBF16>& x);

template <>
__device__ __forceinline__ float dot_head<false>(unsigned w0, const XChunk<false>& x) {
    return fp4x2_to_f32<0>(w0).x * x.v[0];
}
template <>
__device__ __forceinline__ float dot_tail<false>(float part, unsigned w0, unsigned w1, const XChunk<false>& x) {
    f32x2 a = fp4x2_to_f32<0>(w0), b = fp4x2_to_f32<1>(w0), c = fp4x2_to_f32<2>(w0), d = fp4x2_to_f32<3>(w0);
    part = __builtin_fmaf(a.y, x.v[1], part);
    part = __builtin_fmaf(b.x, x.v[2], part);
    part = __builtin_fmaf(b.y, x.v[3], part);
    part = __builtin_fmaf(c.x, x.v[4], part);
    part = __builtin_fmaf(c.y, x.v[5], part);
    part = __builtin_fmaf(d.x, x.v[6], part);
    part = __builtin_fmaf(d.y, x.v[7], part);
    a = fp4x2_to_f32<0>(w1), b = fp4x2_to_f32<1>(w1), c = fp4x2_to_f32<2>(w1), d = fp4x2_to_f32<3>(w1);
    part = __builtin_fmaf(a.x, x.v[8], part);
    part = __builtin_fmaf(a.y, x.v[9], part);
    part = __builtin_fmaf(b.x, x.v[10], part);
    part = __builtin_fmaf(b.y, x.v[11], part);
    part = __builtin_fmaf(c.x, x.v[12], part);
    part = __builtin_fmaf(c.y, x.v[13], part);
    part = __builtin_fmaf(d.x, x.v[14], part);
    part = __builtin_fmaf(d.y, x.v[15], part);
    return part;
}

// bf16 activations: both factors are bf16, every product is exact in f32 and the dot
// instruction adds two of them per step (v_dot2c_f32_bf16)
template <>
__device__ __forceinline__ float dot_head<true>(unsigned w0, const XChunk<true>& x) {
    return __builtin_amdgcn_fdot2_f32_bf16(fp4x2_to_bf16<0>(w0), __builtin_bit_cast(bf16x2, x.v[0]), 0.0f, false);
}
template <>
__device__ __forceinline__ float dot_tail<true>(float part, unsigned w0, unsigned w1, const XChunk<true>& x) {
    part = __builtin_amdgcn_fdot2_f32_bf16(fp4x2_to_bf16<1>(w0), __builtin_bit_cast(bf16x2, x.v[1]), part, false);
    part = __builtin_amdgcn_fdot2_f32_bf16(fp4x2_to_bf16<2>(w0), __builtin_bit_cast(bf16x2, x.v[2]), part, false);
    part = __builtin_amdgcn_fdot2_f32_bf16(fp4x2_to_bf16<3>(w0), __builtin_bit_cast(bf16x2, x.v[3]), part, false);
    part = __builtin_amdgcn_fdot2_f32_bf16(fp4x2_to_bf16<0>(w1), __builtin_bit_cast(bf16x2, x.v[4]), part, false);
    part = __builtin_amdgcn_fdot2_f32_bf16(fp4x2_to_bf16<1>(w1), __builtin_bit_cast(bf16x2, x.v[5]), part, false);
    part = __builtin_amdgcn_fdot2_f32_bf16(fp4x2_to_bf16<2>(w1), __builtin_bit_cast(bf16x2, x.v[6]), part, false);
    part = __builtin_amdgcn_fdot2_f32_bf16(fp4x2_to_bf16<3>(w1), __builtin_bit_cast(bf16x2, x.v[7]), part, false);
    return part;
}
template <bool XBF16>
__device__ __forceinline__ float subblock_dot(unsigned w0, unsigned w1, const XChunk<XBF16>& x) {
    return dot_tail<XBF16>(dot_head<XBF16>(w0, x), w0, w1, x);
}

template <int I>
__device__ __forceinline__ float scale_of(const uint4& sc) {  // sub-block I (0..15) of the panel
    return e4m3_to_f32<I & 3>(u4_get(sc, I >> 2));
}

// One 32-column step S of a panel for NR tensors and M activation rows.
template <int NR, int M, bool XBF16, int S>
__device__ __forceinline__ void step(const uint4 (&sc)[NR], const uint4 (&cd)[NR], const void* x, size_t x_off,
                                     size_t x_stride, int m_rows, float (&acc)[NR][M]) {
#pragma unroll
    for (int half = 0; half < 2; half++) {
        XChunk<XBF16> xc[M];
#pragma unroll
        for (int m = 0; m < M; m++)
            if (m < m_rows) xc[m].load(x, (size_t)m * x_stride + x_off + half * 16);
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const unsigned w0 = half ? cd[r].z : cd[r].x, w1 = half ? cd[r].w : cd[r].y;
            const float sf = half ? scale_of<2 * S + 1>(sc[r]) : scale_of<2 * S>(sc[r]);
#pragma unroll
            for (int m = 0; m < M; m++)
                if (m < m_rows) acc[r][m] = __builtin_fmaf(subblock_dot<XBF16>(w0, w1, xc[m]), sf, acc[r][m]);
        }
    }
}

template <int NR, int M, bool XBF16, int S>
struct Steps {
    __device__ __forceinline__ static void run(const uint4 (&sc)[NR], const uint4 (&cd)[NR][CROW_STEPS], const void* x,
                                               size_t x_off, size_t x_stride, int m_rows, int nsteps,
                                               float (&acc)[NR][M]) {
        if (S < nsteps) {
            uint4 c[NR];
#pragma unroll
            for (int r = 0; r < NR; r++) c[r] = cd[r][S];
            step<NR, M, XBF16, S>(sc, c, x, x_off + S * CROW_STEP_COLS, x_stride, m_rows, acc);
        }
        Steps<NR, M, XBF16, S + 1>::run(sc, cd, x, x_off, x_stride, m_rows, nsteps, acc);
    }
    // a whole panel: no per-step test (see panel_full below)
};
template <int NR, int M, bool XBF16>
struct Steps<NR, M, XBF16, CROW_STEPS> {
    __device__ __forceinline__ static void run(const uint4 (&)[NR], const uint4 (&)[NR][CROW_STEPS], const void*, size_t,
                                               size_t, int, int, float (&)[NR][M]) {}
};

// A whole 256-column panel with the activation chunks software-pipelined: the scalar loads of
// sub-block H + 1 are issued before the arithmetic of sub-block H, so their latency is covered by
// 16 * M fused multiply-adds instead of being waited for.
template <int NR, int M, bool XBF16, int H>
struct PanelFull {
    __device__ __forceinline__ static void run(const uint4 (&sc)[NR], const uint4 (&cd)[NR][CROW_STEPS], const void* x, size_t x_off,
                                               size_t x_stride, int m_rows, XChunk<XBF16> (&cur)[M], float (&acc)[NR][M]) {
        // first link of every chain: this is where the wave waits for `cur`; only then are the
        // next sub-block's scalar loads issued (scalar loads return out of order, so a wait covers
        // everything outstanding - issued any earlier they would be waited for here as well)
        float part[NR][M];
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const uint4& c = cd[r][H >> 1];
#pragma unroll
            for (int m = 0; m < M; m++)
                if (m < m_rows) part[r][m] = dot_head<XBF16>((H & 1) ? c.z : c.x, cur[m]);
        }
        __builtin_amdgcn_sched_barrier(0);
        XChunk<XBF16> nxt[M];
        if (H + 1 < 2 * CROW_STEPS) {
#pragma unroll
            for (int m = 0; m < M; m++)
                if (m < m_rows) nxt[m].load(x, (size_t)m * x_stride + x_off + (H + 1) * 16);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const uint4& c = cd[r][H >> 1];
            const unsigned w0 = (H & 1) ? c.z : c.x, w1 = (H & 1) ? c.w : c.y;
            const float sf = scale_of<H>(sc[r]);
#pragma unroll
            for (int m = 0; m < M; m++)
                if (m < m_rows) acc[r][m] = __builtin_fmaf(dot_tail<XBF16>(part[r][m], w0, w1, cur[m]), sf, acc[r][m]);
        }
        PanelFull<NR, M, XBF16, H + 1>::run(sc, cd, x, x_off, x_stride, m_rows, nxt, acc);
    }
};
template <int NR, int M, bool XBF16>
struct PanelFull<NR, M, XBF16, 2 * CROW_STEPS> {
    __device__ __forceinline__ static void run(const uint4 (&)[NR], const uint4 (&)[NR][CROW_STEPS], const void*, size_t, size_t, int,
                                               XChunk<XBF16> (&)[M], float (&)[NR][M]) {}
};

// f32 activations with M >= 3 rows: two 16-value chunks per row (current + prefetched) would need 128
// SGPRs, more than a wave has, and the compiler then parks them in VGPR lanes.  The same chains
// are therefore fed in 8-value chunks (one code word): chunk C is word C & 3 of step C >> 2, i.e.
// half C & 1 of sub-block C >> 1.  Operation order per row is unchanged (one 16-long chain per
// sub-block), so the results are bit-identical to the 16-value form.
struct XHalf {
    float v[8];
    __device__ __forceinline__ void load(const void* x, size_t off) {
        const float* p = (const float*)x + off;
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = p[j];
    }
};
template <int NR, int M, int C>
struct PanelFullHalf {
    __device__ __forceinline__ static void run(const uint4 (&sc)[NR], const uint4 (&cd)[NR][CROW_STEPS], const void* x, size_t x_off,
                                               size_t x_stride, int m_rows, float (&part)[NR][M], float (&acc)[NR][M]) {
        // no software prefetch here: M * 8 SGPRs per chunk is all the scalar file affords next to the
        // addressing; 4 + 8 M instructions per chunk and several waves per SIMD cover the scalar-cache latency
        XHalf cur[M];
#pragma unroll
        for (int m = 0; m < M; m++)
            if (m < m_rows) cur[m].load(x, (size_t)m * x_stride + x_off + C * 8);
#pragma unroll
        for (int r = 0; r < NR; r++) {
            const unsigned word = u4_get(cd[r][C >> 2], C & 3);
            const f32x2 a = fp4x2_to_f32<0>(word), b = fp4x2_to_f32<1>(word), c = fp4x2_to_f32<2>(word), d = fp4x2_to_f32<3>(word);
            const float sf = scale_of<(C >> 1)>(sc[r]);
#pragma unroll
            for (int m = 0; m < M; m++) {
                if (m < m_rows) {
                    float p = (C & 1) ? __builtin_fmaf(a.x, cur[m].v[0], part[r][m]) : a.x * cur[m].v[0];
                    p = __builtin_fmaf(a.y, cur[m].v[1], p);
                    p = __builtin_fmaf(b.x, cur[m].v[2], p);
                    p = __builtin_fmaf(b.y, cur[m].v[3], p);
                    p = __builtin_fmaf(c.x, cur[m].v[4], p);
                    p = __builtin_fmaf(c.y, cur[m].v[5], p);
                    p = __builtin_fmaf(d.x, cur[m].v[6], p);
                    p = __builtin_fmaf(d.y, cur[m].v[7], p);
                    part[r][m] = p;
                    if (C & 1) acc[r][m] = __builtin_fmaf(p, sf, acc[r][m]);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        PanelFullHalf<NR, M, C + 1>::run(sc, cd, x, x_off, x_stride, m_rows, part, acc);
    }
};
template <int NR, int M>
struct PanelFullHalf<NR, M, 32> {
    __device__ __forceinline__ static void run(const uint4 (&)[NR], const uint4 (&)[NR][CROW_STEPS], const void*, size_t, size_t, int,
                                               float (&)[NR][M], float (&)[NR][M]) {}
};

template <int NR>
__device__ __forceinline__ void load_tile(const unsigned char* const (&w)[2], int rt, int panels, int p, int lane,
                                          uint4 (&sc)[NR], uint4 (&cd)[NR][CROW_STEPS]) {
#pragma unroll
    for (int r = 0; r < NR; r++) {
        const uint4* t = (const uint4*)(w[r] + ((size_t)rt * panels + p) * CROW_TILE_BYTES) + lane;
        sc[r] = stream_load(t);
#pragma unroll
        for (int s = 0; s < CROW_STEPS; s++) cd[r][s] = stream_load(t + 64 * (s + 1));
    }
}

template <int NR, int M, bool XBF16>
__device__ __forceinline__ void panel_compute(const uint4 (&sc)[NR], const uint4 (&cd)[NR][CROW_STEPS], int p, int k_dim,
                                              const void* x, size_t x_stride, int m_rows, float (&acc)[NR][M]) {
    const int left = (k_dim - p * CROW_PANEL_COLS) / CROW_STEP_COLS;
    if (left >= CROW_STEPS && !XBF16 && M >= 3) {
        float part[NR][M];
        PanelFullHalf<NR, M, 0>::run(sc, cd, x, (size_t)p * CROW_PANEL_COLS, x_stride, m_rows, part, acc);
    } else if (left >= CROW_STEPS) {
        XChunk<XBF16> first[M];
#pragma unroll
        for (int m = 0; m < M; m++)
            if (m < m_rows) first[m].load(x, (size_t)m * x_stride + (size_t)p * CROW_PANEL_COLS);
        PanelFull<NR, M, XBF16, 0>::run(sc, cd, x, (size_t)p * CROW_PANEL_COLS, x_stride, m_rows, first, acc);
    } else {
        Steps<NR, M, XBF16, 0>::run(sc, cd, x, (size_t)p * CROW_PANEL_COLS, x_stride, m_rows, left, acc);
    }
}

// Ordering point of the cross-block hand-over.  Every access to the shared partials and counters
// is a device-scope atomic (store / load / add carry the device-coherence bits, so each one is
// performed at the level all compute dies share); what is left to guarantee is program order
// between them, which a wait for this wave's outstanding memory operations gives: the partial
// stores are acknowledged before the arrival counter is bumped, and the counter's value is back
// before any partial is read.  No cache-wide write-back or invalidate is issued: device-scope
// fences were measured at tens of microseconds per launch here because every block pays one.
__device__ __forceinline__ void device_order() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("" ::: "memory");
}

// acc[r][m] = sum over panels p = p0, p0 + stride, ... of the 64-row tile `rt` of tensor r against
// activation row m: the per-lane (= per-row) partial dot product of one wave.  One register buffer
// per wave; loads and arithmetic of different waves overlap through occupancy (about 52 VGPRs).
template <int NR, int M, bool XBF16>
__device__ __forceinline__ void tile_accumulate(const unsigned char* const (&w)[2], int rt, int panels, int p0, int stride,
                                                int k_dim, const void* x, size_t x_stride, int m_rows, float (&acc)[NR][M]) {
    const int lane = lane_id();
#pragma unroll
    for (int r = 0; r < NR; r++)
#pragma unroll
        for (int m = 0; m < M; m++) acc[r][m] = 0.0f;
    for (int p = p0; p < panels; p += stride) {
        uint4 sc[NR], cd[NR][CROW_STEPS];
        load_tile<NR>(w, rt, panels, p, lane, sc, cd);
        panel_compute<NR, M, XBF16>(sc, cd, p, k_dim, x, x_stride, m_rows, acc);
    }
}

typedef __attribute__((address_space(1))) float* gfloat_p;
typedef __attribute__((address_space(1))) unsigned* guint_p;
typedef __attribute__((address_space(1))) int* gint_p;

// The body every GEMV entry point runs.  The caller has already offset the pointers in `a` for
// its token group / combo `z`, which only indexes the workspace here.  `red` is the block's LDS
// hand-over buffer of (W - 1) * NR * M * 64 floats (RED_FLOATS of them are there).
template <int NR, int M, bool XBF16, int EPI, int RED_FLOATS>
__device__ __forceinline__ void gemv_body(const GemvArgs& a, unsigned z, float* red, const Workspace& ws) {
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), waves = block_threads() >> 6;  // wave-uniform on purpose
    const int slice = (int)blockIdx.x, slices = (int)gridDim.x;
    const int rt = (int)blockIdx.y;
    const int row_tiles = (int)gridDim.y;
    const int panels = (a.k_dim + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS;
    const int m_rows = a.m < M ? a.m : M;
    const unsigned tile_id = z * (unsigned)row_tiles + (unsigned)rt;

    float acc[NR][M];
    tile_accumulate<NR, M, XBF16>(a.w, rt, panels, slice * waves + wave, slices * waves, a.k_dim, a.x, a.x_stride, m_rows, acc);

    // waves of the block -> wave 0, in wave order
    if (waves > 1) {
        if ((waves - 1) * NR * M * 64 > RED_FLOATS) {  // uniform: the launch does not fit this kernel
            if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
            return;
        }
        if (wave > 0) {
#pragma unroll
            for (int r = 0; r < NR; r++)
#pragma unroll
                for (int m = 0; m < M; m++)
                    if (m < m_rows) red[((wave - 1) * NR * M + r * M + m) * 64 + lane] = acc[r][m];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int w = 1; w < waves; w++) {
#pragma unroll
            for (int r = 0; r < NR; r++)
#pragma unroll
                for (int m = 0; m < M; m++)
                    if (m < m_rows) acc[r][m] += red[((w - 1) * NR * M + r * M + m) * 64 + lane];
        }
    }

    // slices of the row tile -> the last one to arrive, in slice order
    if (slices > 1) {
        const size_t need = ((size_t)tile_id + 1) * slices * (NR * M) * 64;
        if (need > ws.partial_floats || tile_id >= ws.counter_slots) {
            if (lane == 0) atomicOr(ws.status, STATUS_WORKSPACE_TOO_SMALL);
            return;
        }
        gfloat_p base = (gfloat_p)ws.partials + (size_t)tile_id * slices * (NR * M) * 64;
        gfloat_p mine = base + (size_t)slice * (NR * M) * 64;
        guint_p counter = (guint_p)ws.counters + tile_id;
#pragma unroll
        for (int r = 0; r < NR; r++)
#pragma unroll
            for (int m = 0; m < M; m++)
                if (m < m_rows) __hip_atomic_store(mine + (r * M + m) * 64 + lane, acc[r][m], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        device_order();
        unsigned arrived = 0;
        if (lane == 0) arrived = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        arrived = __builtin_amdgcn_readfirstlane(arrived);
        if (arrived != (unsigned)slices - 1) return;
        device_order();
#pragma unroll
        for (int r = 0; r < NR; r++)
#pragma unroll
            for (int m = 0; m < M; m++) acc[r][m] = 0.0f;
        // up to PB slices' loads in flight at a time, added in slice order
        constexpr int PB = (NR * M <= 2) ? 16 : 8;
        for (int s0 = 0; s0 < slices; s0 += PB) {
            float t[PB][NR * M];
#pragma unroll
            for (int j = 0; j < PB; j++) {
                gfloat_p q = base + (size_t)(s0 + j) * (NR * M) * 64 + lane;
#pragma unroll
                for (int i = 0; i < NR * M; i++)
                    t[j][i] = (s0 + j < slices && (i % M) < m_rows) ? __hip_atomic_load(q + i * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.0f;
            }
#pragma unroll
            for (int j = 0; j < PB; j++) {
                if (s0 + j < slices) {
#pragma unroll
                    for (int r = 0; r < NR; r++)
#pragma unroll
                        for (int m = 0; m < M; m++) acc[r][m] += t[j][r * M + m];
                }
            }
        }
        if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    const int row = rt * CROW_TILE_ROWS + lane;
    if (EPI == EPI_SCALE && a.argmax_out != nullptr) {
        // fused head, stage 1: logits out and one (value, index) candidate per row tile into the
        // workspace, plain stores, no waiting (a wave that lingers for an arrival protocol keeps
        // its block's slots busy: measured +15 % on the whole launch).  Stage 2 is argmax_tiles.
        const float v = acc[0][0] * a.gs[0][0];
        if (row < a.rows) a.y[row] = v;
        const Best b = wave_best(Best{row < a.rows ? v : -3.0e38f, row < a.rows ? row : 0});
        if ((unsigned)row_tiles > ws.am_slots) {
            if (lane == 0) atomicOr(ws.status, STATUS_WORKSPACE_TOO_SMALL);
            return;
        }
        if (lane == 0) {
            ws.am_val[rt] = b.v;
            ws.am_idx[rt] = b.i;
        }
        return;
    }
    if (row >= a.rows) return;
    if (EPI == EPI_SCALE) {
        const float gs = a.gs[0][0];
#pragma unroll
        for (int m = 0; m < M; m++)
            if (m < m_rows) a.y[(size_t)m * a.y_stride + row] = acc[0][m] * gs;
    } else {
        const float gg = a.gs[0][0], gu = a.gs[NR - 1][0];
#pragma unroll
        for (int m = 0; m < M; m++)
            if (m < m_rows) a.y[(size_t)m * a.y_stride + row] = silu_mul(acc[0][m] * gg, acc[NR - 1][m] * gu);
    }
}

}  // namespace crow

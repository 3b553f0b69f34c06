// NVFP4 x bf16 batched GEMM on the gfx950 matrix cores: Y[M][N] = X[M][K] W[N][K]^T, M >= 16 token rows.
//
// The reference's prefill projection (engine/src/gen.rs:3922-3924 -> gemm_fp4_dense, engine/src/kernels.rs:
// 533-751) quantises the activations to FP4 and runs Blackwell block-scaled MMA; its structural twin
// glm5_gemm_fp4_tc (engine/src/kernels_glm5_moe.cu:349-449) decodes the weights losslessly to 16-bit
// tiles and runs a plain tensor-core MMA with f32 accumulation and gs in the epilogue.  This kernel
// is the CDNA4 form of the latter: weights decode to EXACT bf16 (e2m1 * ue4m3 has at most 6
// significant bits), X is bf16, products are exact in f32, v_mfma_f32_32x32x16_bf16 accumulates.
//
// Data flow.  A block is 4 waves; wave w owns row tile 4 * blockIdx.x + w (64 weight rows) and all
// of the block's MT = 32 * TB token rows.  Per 256-column panel:
//   * every wave loads its own 9216-byte weight tile straight into registers (the GEMV's loads);
//   * the block stages X[m0 .. m0 + MT][panel] into LDS (row stride 528 B: conflict-free b128 reads);
//   * per 16-column sub-block the two code words a lane holds for ITS row are exchanged between the
//     wave halves with v_permlane32_swap, which turns "lane = row, 16 columns" into the MFMA operand
//     shape "lane % 32 = row, lane / 32 = which 8 columns" for rows 0..31 and rows 32..63 at once -
//     on the 4-bit codes, before any decode; each half then decodes 8 values (cvt to f32, times the
//     sub-block scale, keep the high 16 bits: exact) and feeds TB MFMAs per row half.
// The weight rows ride on the MFMA's N side and the tokens on its M side, so a lane's 16 results
// are 16 tokens of one weight row and every store instruction writes 128 contiguous bytes of Y.
#pragma once
#include "device_common.h"

namespace crow {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

#define CROW_GEMM_XS_STRIDE 264  // bf16 elements per staged X row (256 + 8 of padding)

// 8 codes (one word) times a sub-block scale -> 8 exact bf16 values, as an MFMA operand
__device__ __forceinline__ bf16x8 decode8_bf16(unsigned codes, float scale) {
    const f32x2 a = fp4x2_to_f32<0>(codes), b = fp4x2_to_f32<1>(codes), c = fp4x2_to_f32<2>(codes), d = fp4x2_to_f32<3>(codes);
    u32x4 r;
    // byte selector 0x07060302: high halves of (hi, lo) -> {lo[31:16], hi[31:16]}
    r.x = __builtin_amdgcn_perm(__float_as_uint(a.y * scale), __float_as_uint(a.x * scale), 0x07060302u);
    r.y = __builtin_amdgcn_perm(__float_as_uint(b.y * scale), __float_as_uint(b.x * scale), 0x07060302u);
    r.z = __builtin_amdgcn_perm(__float_as_uint(c.y * scale), __float_as_uint(c.x * scale), 0x07060302u);
    r.w = __builtin_amdgcn_perm(__float_as_uint(d.y * scale), __float_as_uint(d.x * scale), 0x07060302u);
    return __builtin_bit_cast(bf16x8, r);
}

template <int SB>
__device__ __forceinline__ float scale_byte(unsigned word) {
    return e4m3_to_f32<SB & 3>(word);
}

// one 16-column sub-block SB (0..15) of the panel
template <int TB, int SB>
__device__ __forceinline__ void gemm_subblock(const uint4& cd, unsigned sc_lo, unsigned sc_hi, const __bf16* xs_lane,
                                              f32x16 (&acc)[2][TB]) {
    const unsigned d0 = (SB & 1) ? cd.z : cd.x, d1 = (SB & 1) ? cd.w : cd.y;
    // after the swap: .x = codes of rows 0..31 (lanes 0..31: columns 0..7, lanes 32..63: columns 8..15),
    //                 .y = the same for rows 32..63
    const u32x2 sw = __builtin_amdgcn_permlane32_swap(d0, d1, false, false);
    const bf16x8 w_lo = decode8_bf16(sw.x, scale_byte<SB>(sc_lo));
    const bf16x8 w_hi = decode8_bf16(sw.y, scale_byte<SB>(sc_hi));
#pragma unroll
    for (int tb = 0; tb < TB; tb++) {
        const bf16x8 xv = *(const bf16x8*)(xs_lane + tb * 32 * CROW_GEMM_XS_STRIDE + SB * 16);
        acc[0][tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xv, w_lo, acc[0][tb], 0, 0, 0);
        acc[1][tb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xv, w_hi, acc[1][tb], 0, 0, 0);
    }
}

template <int TB, int SB>
struct GemmPanel {
    __device__ __forceinline__ static void run(const uint4 (&cd)[CROW_STEPS], const unsigned (&lo)[4], const unsigned (&hi)[4],
                                               const __bf16* xs_lane, f32x16 (&acc)[2][TB]) {
        gemm_subblock<TB, SB>(cd[SB >> 1], lo[SB >> 2], hi[SB >> 2], xs_lane, acc);
        // keep sub-blocks in program order: a wave's decode then overlaps the OTHER resident waves' MFMAs,
        // and the register count stays low enough for several waves per SIMD
        __builtin_amdgcn_sched_barrier(0);
        GemmPanel<TB, SB + 1>::run(cd, lo, hi, xs_lane, acc);
    }
};
template <int TB>
struct GemmPanel<TB, 16> {
    __device__ __forceinline__ static void run(const uint4 (&)[CROW_STEPS], const unsigned (&)[4], const unsigned (&)[4], const __bf16*,
                                               f32x16 (&)[2][TB]) {}
};

template <int TB>
__device__ __forceinline__ void gemm_body(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                          const float* __restrict__ gs_ptr, float* __restrict__ y, int k_dim, int rows, int m_total,
                                          __bf16* xs) {
    constexpr int MT = 32 * TB;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int row_tiles = (rows + CROW_TILE_ROWS - 1) / CROW_TILE_ROWS;
    const int rt = (int)blockIdx.x * 4 + wave;
    const bool has_rows = rt < row_tiles;  // wave-uniform; idle waves still join the barriers
    const int m0 = (int)blockIdx.y * MT;
    const int panels = (k_dim + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS;

    f32x16 acc[2][TB];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int tb = 0; tb < TB; tb++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[h][tb][i] = 0.0f;

    // this lane's fixed read position in the staged X tile: token lane % 32, columns 8 * (lane / 32) ..
    const __bf16* xs_lane = xs + (lane & 31) * CROW_GEMM_XS_STRIDE + (lane >> 5) * 8;

    // two register buffers for the weight tile: panel p + 1 is in flight while panel p is multiplied
    uint4 scA = make_uint4(0, 0, 0, 0), cdA[CROW_STEPS], scB = make_uint4(0, 0, 0, 0), cdB[CROW_STEPS];
#pragma unroll
    for (int s = 0; s < CROW_STEPS; s++) cdA[s] = cdB[s] = make_uint4(0, 0, 0, 0);
    const uint4* wt = (const uint4*)(w + (size_t)rt * panels * CROW_TILE_BYTES) + lane;
    auto load_w = [&](int p, uint4& sc, uint4 (&cd)[CROW_STEPS]) {
        if (has_rows && p < panels) {
            const uint4* t = wt + (size_t)p * (CROW_TILE_BYTES / 16);
            sc = stream_load(t);
#pragma unroll
            for (int s = 0; s < CROW_STEPS; s++) cd[s] = stream_load(t + 64 * (s + 1));
        }
    };
    auto stage_x = [&](int p) {
        // X[m0 .. m0 + MT][256 p .. 256 p + 255] (zero beyond M and K): MT * 32 chunks of 16 bytes
        __syncthreads();  // the previous panel's reads are done
        for (int c = (int)threadIdx.x; c < MT * 32; c += 256) {
            const int r = c >> 5, q = c & 31;
            const int m = m0 + r, k = p * CROW_PANEL_COLS + q * 8;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m < m_total && k < k_dim) v = *(const uint4*)(x + (size_t)m * k_dim + k);
            *(uint4*)(xs + r * CROW_GEMM_XS_STRIDE + q * 8) = v;
        }
        __syncthreads();
    };
    auto multiply = [&](const uint4& sc, const uint4 (&cd)[CROW_STEPS]) {
        // scale words of rows 0..31 / 32..63 in both wave halves
        unsigned lo[4], hi[4];
        const u32x2 a = __builtin_amdgcn_permlane32_swap(sc.x, sc.x, false, false);
        const u32x2 b = __builtin_amdgcn_permlane32_swap(sc.y, sc.y, false, false);
        const u32x2 c = __builtin_amdgcn_permlane32_swap(sc.z, sc.z, false, false);
        const u32x2 d = __builtin_amdgcn_permlane32_swap(sc.w, sc.w, false, false);
        lo[0] = a.x; lo[1] = b.x; lo[2] = c.x; lo[3] = d.x;
        hi[0] = a.y; hi[1] = b.y; hi[2] = c.y; hi[3] = d.y;
        GemmPanel<TB, 0>::run(cd, lo, hi, xs_lane, acc);
    };
    if (TB <= 2) {
        load_w(0, scA, cdA);
        for (int p = 0; p < panels; p += 2) {
            stage_x(p);
            load_w(p + 1, scB, cdB);
            multiply(scA, cdA);
            if (p + 1 >= panels) break;
            stage_x(p + 1);
            load_w(p + 2, scA, cdA);
            multiply(scB, cdB);
        }
    } else {  // 128 tokens: the accumulators leave no room for a second weight buffer; two blocks per CU overlap instead
        for (int p = 0; p < panels; p++) {
            load_w(p, scA, cdA);
            stage_x(p);
            multiply(scA, cdA);
        }
    }
    if (!has_rows) return;

    // acc[h][tb][v]: token 32 tb + 8 (v / 4) + 4 (lane / 32) + v % 4, weight row 64 rt + 32 h + lane % 32
    const float gs = gs_ptr[0];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int n = rt * CROW_TILE_ROWS + h * 32 + (lane & 31);
        if (n >= rows) continue;
#pragma unroll
        for (int tb = 0; tb < TB; tb++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + tb * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (m < m_total) y[(size_t)m * rows + n] = acc[h][tb][v] * gs;
            }
    }
}

// M <= 32 token rows: the product is bandwidth-bound and needs every CU streaming, so a block is ONE row
// tile whose panels are dealt to its 4 waves (wave w: panels w, w + 4, ...).  Each wave stages its
// own X panel in its own LDS region and reads it back itself: no block barrier in the loop.  The
// four partial tiles are added in wave order through LDS at the end (deterministic).
__device__ __forceinline__ void gemm_small_body(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                                const float* __restrict__ gs_ptr, float* __restrict__ y, int k_dim, int rows,
                                                int m_total, __bf16* xs_all) {
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int rt = (int)blockIdx.x;
    const int panels = (k_dim + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS;
    __bf16* xs = xs_all + wave * (32 * CROW_GEMM_XS_STRIDE);
    const __bf16* xs_lane = xs + (lane & 31) * CROW_GEMM_XS_STRIDE + (lane >> 5) * 8;

    f32x16 acc[2][1];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[h][0][i] = 0.0f;

    uint4 scA = make_uint4(0, 0, 0, 0), cdA[CROW_STEPS], scB = make_uint4(0, 0, 0, 0), cdB[CROW_STEPS];
#pragma unroll
    for (int s = 0; s < CROW_STEPS; s++) cdA[s] = cdB[s] = make_uint4(0, 0, 0, 0);
    const uint4* wt = (const uint4*)(w + (size_t)rt * panels * CROW_TILE_BYTES) + lane;
    auto load_w = [&](int p, uint4& sc, uint4 (&cd)[CROW_STEPS]) {
        if (p < panels) {
            const uint4* t = wt + (size_t)p * (CROW_TILE_BYTES / 16);
            sc = stream_load(t);
#pragma unroll
            for (int s = 0; s < CROW_STEPS; s++) cd[s] = stream_load(t + 64 * (s + 1));
        }
    };
    auto stage_x = [&](int p) {  // 32 tokens x 256 columns = 1024 chunks of 16 bytes, 16 per lane; wave-private
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int c = i * 64 + lane, r = c >> 5, q = c & 31;
            const int k = p * CROW_PANEL_COLS + q * 8;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (r < m_total && k < k_dim) v = *(const uint4*)(x + (size_t)r * k_dim + k);
            *(uint4*)(xs + r * CROW_GEMM_XS_STRIDE + q * 8) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    auto multiply = [&](const uint4& sc, const uint4 (&cd)[CROW_STEPS]) {
        unsigned lo[4], hi[4];
        const u32x2 a = __builtin_amdgcn_permlane32_swap(sc.x, sc.x, false, false);
        const u32x2 b = __builtin_amdgcn_permlane32_swap(sc.y, sc.y, false, false);
        const u32x2 c = __builtin_amdgcn_permlane32_swap(sc.z, sc.z, false, false);
        const u32x2 d = __builtin_amdgcn_permlane32_swap(sc.w, sc.w, false, false);
        lo[0] = a.x; lo[1] = b.x; lo[2] = c.x; lo[3] = d.x;
        hi[0] = a.y; hi[1] = b.y; hi[2] = c.y; hi[3] = d.y;
        GemmPanel<1, 0>::run(cd, lo, hi, xs_lane, acc);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the tile is read before the next stage overwrites it
        __builtin_amdgcn_wave_barrier();
    };
    load_w(wave, scA, cdA);
    for (int p = wave; p < panels; p += 8) {
        stage_x(p);
        load_w(p + 4, scB, cdB);
        multiply(scA, cdA);
        if (p + 4 >= panels) break;
        stage_x(p + 4);
        load_w(p + 8, scA, cdA);
        multiply(scB, cdB);
    }
    // waves 1..3 -> wave 0 through LDS (each wave's own region is free now), added in wave order
    float* red = (float*)xs;
    if (wave > 0) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int v = 0; v < 16; v++) red[(h * 16 + v) * 64 + lane] = acc[h][0][v];
    }
    __syncthreads();
    if (wave > 0) return;
    for (int ww = 1; ww < 4; ww++) {
        const float* q = (const float*)(xs_all + ww * (32 * CROW_GEMM_XS_STRIDE));
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[h][0][v] += q[(h * 16 + v) * 64 + lane];
    }
    const float gs = gs_ptr[0];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int n = rt * CROW_TILE_ROWS + h * 32 + (lane & 31);
        if (n >= rows) continue;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
            if (m < m_total) y[(size_t)m * rows + n] = acc[h][0][v] * gs;
        }
    }
}

}  // namespace crow

// Y[M][rows] f32 = X[M][k_dim] bf16 times the tiled NVFP4 tensor, times gs.  The argument list is
// gemm_fp4_dense's (engine/src/kernels.rs:533-541) without the quantised-activation buffer: x is bf16.
// grid (ceil(row_tiles / 4), ceil(M / MT)), block 256, MT = 32 / 64 / 128 for the three entry points.
#define CROW_GEMM_ENTRY(NAME, TB)                                                                                             \
    extern "C" __global__ void __launch_bounds__(256, 2) NAME(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x, \
                                                           const float* __restrict__ gs_ptr, float* __restrict__ y,            \
                                                           const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,    \
                                                           const int* __restrict__ m_p) {                                      \
        __shared__ __attribute__((aligned(16))) __bf16 xs[32 * TB * CROW_GEMM_XS_STRIDE];                                      \
        crow::gemm_body<TB>(w, x, gs_ptr, y, *k_dim_p, *rows_p, *m_p, xs);                                                     \
    }
// M <= 32: grid (row_tiles), block 256
extern "C" __global__ void __launch_bounds__(256, 2) gemm_nvfp4_bf16_m32(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                                                         const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                         const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                         const int* __restrict__ m_p) {
    __shared__ __attribute__((aligned(16))) __bf16 xs[4 * 32 * CROW_GEMM_XS_STRIDE];
    crow::gemm_small_body(w, x, gs_ptr, y, *k_dim_p, *rows_p, *m_p, xs);
}
CROW_GEMM_ENTRY(gemm_nvfp4_bf16_m64, 2)
CROW_GEMM_ENTRY(gemm_nvfp4_bf16, 4)

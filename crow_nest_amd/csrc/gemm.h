// NVFP4 x bf16 batched GEMM on the gfx950 matrix cores: Y[M][N] = X[M][K] W[N][K]^T, M > 4 token rows.
//
// The reference's prefill projection (engine/src/gen.rs:3922-3924 -> gemm_fp4_dense, engine/src/kernels.rs:
// 533-751) quantises the activations to FP4 and runs Blackwell block-scaled MMA; its structural twin
// glm5_gemm_fp4_tc (engine/src/kernels_glm5_moe.cu:349-449) decodes the weights losslessly to 16-bit
// tiles and runs a plain tensor-core MMA with f32 accumulation and gs in the epilogue.  This kernel
// is the CDNA4 form of the latter: weights decode to EXACT bf16 (e2m1 * ue4m3 has at most 6
// significant bits), X is bf16, products are exact in f32, v_mfma_f32_16x16x32_bf16 accumulates.
//
// Data flow.  A wave owns a 64-row weight tile - four 16-row strips of the layout - per 256-column panel and MT = 16 * TBK token
// rows.  Per panel:
//   * the wave loads the panel's group of each of its four strips (4 x 2304 bytes) straight into registers; every code
//     dword is the B operand of one "unit" (16 weight rows x 32 columns, layout.h) as it stands;
//   * X[m0 .. m0 + MT][panel] is staged in LDS (row stride 528 B) and read back as A operands, 16 token rows x
//     32 columns per 16-byte-per-lane read, each used for the four row groups of the tile;
//   * per unit a lane turns its 8 codes into 8 bf16 values times the sub-block scale (cvt to f32, multiply,
//     keep the high 16 bits: exact) and feeds TBK matrix instructions.
// The weight rows ride on the N side and the tokens on the M side, so a lane's 4 results of an instruction are
// 4 tokens of one weight row and a store instruction writes four 64-byte runs of Y.
#pragma once
#include "gemv.h"

namespace crow {

#define CROW_GEMM_XS_STRIDE 264  // bf16 elements per staged X row (256 + 8 of padding)

// 8 codes (one word) times a sub-block scale -> 8 exact bf16 values, as an MFMA operand
__device__ __forceinline__ bf16x8 decode8_scaled(unsigned codes, float scale) {
    const f32x2 a = fp4x2_to_f32<0>(codes), b = fp4x2_to_f32<1>(codes), c = fp4x2_to_f32<2>(codes), d = fp4x2_to_f32<3>(codes);
    u32x4 r;
    // byte selector 0x07060302: high halves of (hi, lo) -> {lo[31:16], hi[31:16]}
    r.x = __builtin_amdgcn_perm(__float_as_uint(a.y * scale), __float_as_uint(a.x * scale), 0x07060302u);
    r.y = __builtin_amdgcn_perm(__float_as_uint(b.y * scale), __float_as_uint(b.x * scale), 0x07060302u);
    r.z = __builtin_amdgcn_perm(__float_as_uint(c.y * scale), __float_as_uint(c.x * scale), 0x07060302u);
    r.w = __builtin_amdgcn_perm(__float_as_uint(d.y * scale), __float_as_uint(d.x * scale), 0x07060302u);
    return __builtin_bit_cast(bf16x8, r);
}

#define CROW_TILE_ROWS 64    // four strips
#define CROW_PANEL_COLS 256  // one group per strip
// the registers of one panel of a 64-row tile: per strip J one scale dword and two code quadwords
struct PanelRegs {
    unsigned sc[4];
    uint4 cd[4][2];
};
// `w` = the tensor, `strips` / `groups` its strip and group counts; strips beyond the tensor re-read the last one (their rows
// are never stored)
__device__ __forceinline__ void load_panel(const unsigned char* w, int rt, int strips, int groups, int p, int lane, PanelRegs& r) {
#pragma unroll
    for (int J = 0; J < 4; J++) {
        const int strip = 4 * rt + J < strips ? 4 * rt + J : strips - 1;
        const unsigned char* g = w + ((size_t)strip * groups + p) * CROW_GROUP_BYTES;
        r.sc[J] = stream_load_u32((const unsigned*)g + lane);
        r.cd[J][0] = stream_load((const uint4*)(g + CROW_GROUP_SCALE_BYTES) + lane);
        r.cd[J][1] = stream_load((const uint4*)(g + CROW_GROUP_SCALE_BYTES + 1024) + lane);
    }
}

// The panel's scale bytes as the GEMM needs them.  A lane (g, n) holds, for each strip, the scales of segment g & 1 of every
// pair, sub-block half g >> 1 (layout.h); the other segment's are in the neighbouring 16-lane group.  After the exchange `even`
// holds the word of the even group of each 32-lane half in both groups, `odd` that of the odd one.
struct TileScales {
    unsigned even[4], odd[4];
    __device__ __forceinline__ void set(const unsigned (&sc)[4]) {
#pragma unroll
        for (int J = 0; J < 4; J++) {
            const u32x2 sw = __builtin_amdgcn_permlane16_swap(sc[J], sc[J], false, false);
            even[J] = sw.x;
            odd[J] = sw.y;
        }
    }
    // scale of this lane's operand of unit (strip J, segment S of the panel): pair S / 2, segment S % 2
    template <int S, int J>
    __device__ __forceinline__ float get() const {
        return e4m3_to_f32<(S >> 1)>((S & 1) ? odd[J] : even[J]);
    }
};

// one 32-column segment S of the panel: four units, TBK token blocks each
template <int TBK, int S>
__device__ __forceinline__ void gemm_segment(const PanelRegs& r, const TileScales& ts, const __bf16* xs_lane, f32x4 (&acc)[TBK][4]) {
    bf16x8 A[TBK];
#pragma unroll
    for (int tb = 0; tb < TBK; tb++) A[tb] = *(const bf16x8*)(xs_lane + tb * 16 * CROW_GEMM_XS_STRIDE + S * 32);
#define CROW_GEMM_UNIT(J)                                                                                      \
    {                                                                                                          \
        const bf16x8 B = decode8_scaled(u4_get(r.cd[J][S >> 2], S & 3), ts.get<S, J>());                       \
        _Pragma("unroll") for (int tb = 0; tb < TBK; tb++)                                                     \
            acc[tb][J] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[tb], B, acc[tb][J], 0, 0, 0);               \
    }
    CROW_GEMM_UNIT(0) CROW_GEMM_UNIT(1) CROW_GEMM_UNIT(2) CROW_GEMM_UNIT(3)
#undef CROW_GEMM_UNIT
}

template <int TBK>
__device__ __forceinline__ void gemm_panel(const PanelRegs& r, const __bf16* xs_lane, f32x4 (&acc)[TBK][4]) {
    TileScales ts;
    ts.set(r.sc);
    gemm_segment<TBK, 0>(r, ts, xs_lane, acc);
    gemm_segment<TBK, 1>(r, ts, xs_lane, acc);
    gemm_segment<TBK, 2>(r, ts, xs_lane, acc);
    gemm_segment<TBK, 3>(r, ts, xs_lane, acc);
    gemm_segment<TBK, 4>(r, ts, xs_lane, acc);
    gemm_segment<TBK, 5>(r, ts, xs_lane, acc);
    gemm_segment<TBK, 6>(r, ts, xs_lane, acc);
    gemm_segment<TBK, 7>(r, ts, xs_lane, acc);
}

// acc[tb][j][r] of lane (g, n): token m0 + 16 tb + 4 g + r, weight row 64 rt + 16 j + n
template <int TBK>
__device__ __forceinline__ void gemm_store(const f32x4 (&acc)[TBK][4], float gs, float* __restrict__ y, int rt, int m0, int rows, int m_total,
                                           int lane) {
    const int g = lane >> 4, n = lane & 15;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int col = rt * CROW_TILE_ROWS + 16 * j + n;
        if (col >= rows) continue;
#pragma unroll
        for (int tb = 0; tb < TBK; tb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int m = m0 + 16 * tb + 4 * g + r;
                if (m < m_total) y[(size_t)m * rows + col] = acc[tb][j][r] * gs;
            }
    }
}

// Token blocks of 16 TBK rows: a block is ONE row tile and one token block (blockIdx.y) whose panels are dealt to
// its W waves (wave w: panels w, w + W, ...; W = 4 as launched: 8 measured slower at M = 16), so that even a small M puts
// every SIMD to work.  Each wave stages
// its own X panel in its own LDS region and reads it back itself: no block barrier in the loop.  The
// four partial tiles are added in wave order through LDS at the end (deterministic).
template <int TBK>
__device__ __forceinline__ void gemm_small_body(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                                const float* __restrict__ gs_ptr, float* __restrict__ y, int k_dim, int rows,
                                                int m_total, __bf16* xs_all) {
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int rt = (int)blockIdx.x, m0 = 32 * (int)blockIdx.y;
    const int panels = (k_dim + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS;
    if (rt * CROW_TILE_ROWS >= rows || m0 >= m_total) return;  // a grid larger than the problem: the whole block leaves
    const int waves = block_threads() >> 6;  // 16 TBK staged rows per wave
    const int slice = (int)blockIdx.z, slices = (int)gridDim.z;  // the panels may also be dealt over blocks (workspace hand-over)
    __bf16* xs = xs_all + wave * (16 * TBK * CROW_GEMM_XS_STRIDE);
    const __bf16* xs_lane = xs + (lane & 15) * CROW_GEMM_XS_STRIDE + (lane >> 4) * 8;

    f32x4 acc[TBK][4];
#pragma unroll
    for (int tb = 0; tb < TBK; tb++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[tb][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int strips = (rows + CROW_STRIP_ROWS - 1) / CROW_STRIP_ROWS;
    // 16 TBK tokens x 256 columns = 512 TBK chunks of 16 bytes, 8 TBK per lane; wave-private.  Chunk i of this lane: token row
    // 2 i + lane / 32, 8 columns from 8 (lane % 32); its element offset in panel 0 is worked out once (32 bits: checked by
    // the entry points); rows beyond M read row M - 1, whose results are never stored.
    const int xq = (lane & 31) * 8;
    unsigned xoff[8 * TBK];
#pragma unroll
    for (int i = 0; i < 8 * TBK; i++) {
        const int m = m0 + 2 * i + (lane >> 5);
        xoff[i] = (unsigned)(m < m_total ? m : m_total - 1) * (unsigned)k_dim + (unsigned)xq;
    }
    for (int p = slice * waves + wave; p < panels; p += slices * waves) {
        // fetched before the weight loads are issued so that they do not queue behind them
        uint4 xv[8 * TBK];
        const int k0 = p * CROW_PANEL_COLS;
        if (k0 + CROW_PANEL_COLS <= k_dim) {  // uniform
#pragma unroll
            for (int i = 0; i < 8 * TBK; i++) xv[i] = *(const uint4*)(x + (size_t)(xoff[i] + (unsigned)k0));
        } else {  // the last, partial panel: columns beyond K are zeros
#pragma unroll
            for (int i = 0; i < 8 * TBK; i++) {
                xv[i] = make_uint4(0, 0, 0, 0);
                if (k0 + xq < k_dim) xv[i] = *(const uint4*)(x + (size_t)(xoff[i] + (unsigned)k0));
            }
        }
        PanelRegs pr;
        load_panel(w, rt, strips, panels, p, lane, pr);
#pragma unroll
        for (int i = 0; i < 8 * TBK; i++) {
            const int c = i * 64 + lane, r = c >> 5, q = c & 31;
            *(uint4*)(xs + r * CROW_GEMM_XS_STRIDE + q * 8) = xv[i];
        }
        __builtin_amdgcn_wave_barrier();
        gemm_panel<TBK>(pr, xs_lane, acc);
        __builtin_amdgcn_wave_barrier();  // the tile is read before the next stage overwrites it
    }
    // the other waves -> wave 0 through LDS (each wave's own region is free now), added in wave order
    float* red = (float*)xs;
    if (wave > 0) {
#pragma unroll
        for (int tb = 0; tb < TBK; tb++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) red[((tb * 4 + j) * 4 + r) * 64 + lane] = acc[tb][j][r];
    }
    __syncthreads();
    if (wave > 0) return;
    for (int ww = 1; ww < waves; ww++) {
        const float* q = (const float*)(xs_all + ww * (16 * TBK * CROW_GEMM_XS_STRIDE));
#pragma unroll
        for (int tb = 0; tb < TBK; tb++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[tb][j][r] += q[((tb * 4 + j) * 4 + r) * 64 + lane];
    }
    if (slices > 1) {  // slices of the row tile -> the block that arrives last, in slice order (the GEMV's protocol)
        float v[16 * TBK];
#pragma unroll
        for (int tb = 0; tb < TBK; tb++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) v[(tb * 4 + j) * 4 + r] = acc[tb][j][r];
        if (!slice_hand_over<16 * TBK>(v, (unsigned)blockIdx.y * gridDim.x + blockIdx.x, slice, slices, g_ws, lane)) return;
#pragma unroll
        for (int tb = 0; tb < TBK; tb++)
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[tb][j][r] = v[(tb * 4 + j) * 4 + r];
    }
    gemm_store<TBK>(acc, gs_ptr[0], y, rt, m0, rows, m_total, lane);
}

// Shared X: block = 4 waves; wave w owns row tile 4 * blockIdx.x + w and all of the block's MT = 16 * TBK token rows, staged
// once in LDS for the four row tiles.  The memory traffic of panel p + 1 is in flight while panel p is computed: the next
// weight tile waits in a second register set and the next X tile in registers, written to the OTHER LDS buffer after the
// compute, so one block barrier per panel (these kernels run one or two waves per SIMD: nothing else hides the latency).
template <int TBK>
__device__ __forceinline__ void gemm_pipe_body(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                               const float* __restrict__ gs_ptr, float* __restrict__ y, int k_dim, int rows, int m_total,
                                               __bf16* xs2) {
    constexpr int MT = 16 * TBK;
    constexpr int XCH = MT * 32 / 256;  // 16-byte chunks of an X tile per thread
    constexpr int XBUF = MT * CROW_GEMM_XS_STRIDE;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int row_tiles = (rows + CROW_TILE_ROWS - 1) / CROW_TILE_ROWS;
    const int rt = (int)blockIdx.x * 4 + wave;
    const bool has_rows = rt < row_tiles;  // wave-uniform; idle waves still stage X and join the barriers
    const int m0 = (int)blockIdx.y * MT;
    const int panels = (k_dim + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS;

    f32x4 acc[TBK][4];
#pragma unroll
    for (int tb = 0; tb < TBK; tb++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[tb][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int strips = (rows + CROW_STRIP_ROWS - 1) / CROW_STRIP_ROWS;
    auto load_w = [&](int p, PanelRegs& r) { load_panel(w, has_rows ? rt : 0, strips, panels, p, lane, r); };
    // chunk c = i * 256 + thread: token row c / 32, 8 columns from 8 (c % 32).  The element offset of the chunk in panel 0 is
    // worked out once; rows beyond M read row M - 1 (their results are never stored), so whole panels load without masks.
    const int xq = ((int)threadIdx.x & 31) * 8;
    unsigned xoff[XCH];
#pragma unroll
    for (int i = 0; i < XCH; i++) {
        const int m = m0 + ((i * 256 + (int)threadIdx.x) >> 5);
        xoff[i] = (unsigned)(m < m_total ? m : m_total - 1) * (unsigned)k_dim + (unsigned)xq;
    }
    auto load_x = [&](int p, uint4 (&xv)[XCH]) {
        const int k0 = p * CROW_PANEL_COLS;
        if (k0 + CROW_PANEL_COLS <= k_dim) {  // uniform
#pragma unroll
            for (int i = 0; i < XCH; i++) xv[i] = *(const uint4*)(x + (size_t)(xoff[i] + (unsigned)k0));
        } else {  // the last, partial panel: columns beyond K are zeros (they meet zero weights, but must not be NaN)
#pragma unroll
            for (int i = 0; i < XCH; i++) {
                xv[i] = make_uint4(0, 0, 0, 0);
                if (k0 + xq < k_dim) xv[i] = *(const uint4*)(x + (size_t)(xoff[i] + (unsigned)k0));
            }
        }
    };
    auto store_x = [&](__bf16* xs, const uint4 (&xv)[XCH]) {
#pragma unroll
        for (int i = 0; i < XCH; i++) {
            const int c = i * 256 + (int)threadIdx.x, r = c >> 5, q = c & 31;
            *(uint4*)(xs + r * CROW_GEMM_XS_STRIDE + q * 8) = xv[i];
        }
    };
    const int lane_off = (lane & 15) * CROW_GEMM_XS_STRIDE + (lane >> 4) * 8;

    PanelRegs pr[2];
    uint4 xv[XCH];
    load_x(0, xv);
    load_w(0, pr[0]);
    store_x(xs2, xv);
    __syncthreads();
    // two panels per trip so that the register sets swap roles without copies
    for (int p = 0; p < panels; p += 2) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int pp = p + h;
            if (pp < panels) {
                const bool more = pp + 1 < panels;
                if (more) {
                    load_x(pp + 1, xv);
                    load_w(pp + 1, pr[h ^ 1]);
                }
                gemm_panel<TBK>(pr[h], xs2 + h * XBUF + lane_off, acc);
                if (more) store_x(xs2 + (h ^ 1) * XBUF, xv);
                __syncthreads();  // the other buffer is written, and this one read, by every wave
            }
        }
    }
    if (!has_rows) return;
    gemm_store<TBK>(acc, gs_ptr[0], y, rt, m0, rows, m_total, lane);
}

// Wide shared-X body: a block is EIGHT waves - two per SIMD, so that one wave's operand reads, decode and barrier waits run
// under the other's matrix instructions (with one wave per SIMD all of them are serial: a 256 x 128 x 256 unit takes 5.6 us
// against 3.3 us of issue time) - wave w owns row tile 8 * blockIdx.x + w and all of the block's MT = 16 * TBK token rows,
// staged once in LDS for the eight row tiles.  There is ONE weight register set per wave: the next panel's weights are
// requested when the current panel's last instruction has read them, and the SIMD's other wave hides the latency; the next
// X tile travels through registers into the other LDS buffer as in the body above.  One barrier per panel.
template <int TBK>
__device__ __forceinline__ void gemm_wide_body(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                               const float* __restrict__ gs_ptr, float* __restrict__ y, int k_dim, int rows, int m_total,
                                               __bf16* xs2) {
    constexpr int NW = 8;
    constexpr int MT = 16 * TBK;
    constexpr int NT = 64 * NW;
    constexpr int XCH = MT * 32 / NT;  // 16-byte chunks of an X tile per thread
    static_assert(MT * 32 % NT == 0, "whole chunks per thread");
    constexpr int XBUF = MT * CROW_GEMM_XS_STRIDE;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int row_tiles = (rows + CROW_TILE_ROWS - 1) / CROW_TILE_ROWS;
    const int rt = (int)blockIdx.x * NW + wave;
    const bool has_rows = rt < row_tiles;  // wave-uniform; idle waves still stage X and join the barriers
    const int m0 = (int)blockIdx.y * MT;
    const int panels = (k_dim + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS;
    f32x4 acc[TBK][4];
#pragma unroll
    for (int tb = 0; tb < TBK; tb++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[tb][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int strips = (rows + CROW_STRIP_ROWS - 1) / CROW_STRIP_ROWS;
    // chunk c = i * 512 + thread: token row c / 32, 8 columns from 8 (c % 32); rows beyond M read row M - 1 (never stored)
    const int xq = ((int)threadIdx.x & 31) * 8;
    unsigned xoff[XCH];
#pragma unroll
    for (int i = 0; i < XCH; i++) {
        const int m = m0 + ((i * NT + (int)threadIdx.x) >> 5);
        xoff[i] = (unsigned)(m < m_total ? m : m_total - 1) * (unsigned)k_dim + (unsigned)xq;
    }
    auto load_x = [&](int p, uint4 (&xv)[XCH]) {
        const int k0 = p * CROW_PANEL_COLS;
        const bool full = k0 + CROW_PANEL_COLS <= k_dim;  // uniform
#pragma unroll
        for (int i = 0; i < XCH; i++) {
            xv[i] = make_uint4(0, 0, 0, 0);  // (the last, partial panel: columns beyond K are zeros)
            if (full || k0 + xq < k_dim) xv[i] = *(const uint4*)(x + (size_t)(xoff[i] + (unsigned)k0));
        }
    };
    auto store_x = [&](__bf16* xs, const uint4 (&xv)[XCH]) {
#pragma unroll
        for (int i = 0; i < XCH; i++) {
            const int c = i * NT + (int)threadIdx.x, r = c >> 5, q = c & 31;
            *(uint4*)(xs + r * CROW_GEMM_XS_STRIDE + q * 8) = xv[i];
        }
    };
    const int lane_off = (lane & 15) * CROW_GEMM_XS_STRIDE + (lane >> 4) * 8;
    PanelRegs pr;
    uint4 xv[XCH];
    load_x(0, xv);
    load_panel(w, has_rows ? rt : 0, strips, panels, 0, lane, pr);
    store_x(xs2, xv);
    __syncthreads();
    int h = 0;
    for (int p = 0; p < panels; p++) {
        const bool more = p + 1 < panels;
        if (more) load_x(p + 1, xv);
        gemm_panel<TBK>(pr, xs2 + h * XBUF + lane_off, acc);
        if (more) {
            load_panel(w, has_rows ? rt : 0, strips, panels, p + 1, lane, pr);
            store_x(xs2 + (h ^ 1) * XBUF, xv);
        }
        __syncthreads();  // the other buffer is written, and this one read, by every wave
        h ^= 1;
    }
    if (!has_rows) return;
    gemm_store<TBK>(acc, gs_ptr[0], y, rt, m0, rows, m_total, lane);
}

}  // namespace crow

// Y[M][rows] f32 = X[M][k_dim] bf16 times the tiled NVFP4 tensor, times gs.  The argument list is
// gemm_fp4_dense's (engine/src/kernels.rs:533-541) without the quantised-activation buffer: x is bf16.
// grid (ceil(row_tiles / 4), ceil(M / MT)), block 256, MT = 64 / 128 for the two general entry points.
// token blocks of 32: grid (row_tiles, ceil(M / 32)), block 256 (or fewer whole waves: the waves deal the panels)
extern "C" __global__ void __launch_bounds__(512) gemm_nvfp4_bf16_m32(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                                                         const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                         const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                         const int* __restrict__ m_p) {
    __shared__ __attribute__((aligned(16))) __bf16 xs[4 * 32 * CROW_GEMM_XS_STRIDE];
    const int m = *m_p;
    // four waves stage and reduce in the static LDS below; X is addressed with 32-bit element offsets
    if (m < 1 || block_threads() > 256 || (unsigned long long)m * (unsigned long long)*k_dim_p > 0xffffffffull) {
        if (threadIdx.x == 0) atomicOr(crow::g_ws.status, crow::STATUS_BAD_SHAPE);
        return;
    }
    if (m <= 16) crow::gemm_small_body<1>(w, x, gs_ptr, y, *k_dim_p, *rows_p, m, xs);  // one 16-token block: half the matrix work and staging
    else crow::gemm_small_body<2>(w, x, gs_ptr, y, *k_dim_p, *rows_p, m, xs);
}
// M <= 16: one 16-token block, its panels dealt over grid.z blocks of 4 waves (one panel per wave at K = 5120): grid (row_tiles, 1, S)
extern "C" __global__ void __launch_bounds__(256) gemm_nvfp4_bf16_m16(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                                                       const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                       const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                       const int* __restrict__ m_p) {
    __shared__ __attribute__((aligned(16))) __bf16 xs[4 * 16 * CROW_GEMM_XS_STRIDE];
    const int m = *m_p;
    if (m < 1 || m > 16 || block_threads() > 256 || (unsigned long long)m * (unsigned long long)*k_dim_p > 0xffffffffull) {  // uniform over the launch
        if (threadIdx.x == 0) atomicOr(crow::g_ws.status, crow::STATUS_BAD_SHAPE);
        return;
    }
    crow::gemm_small_body<1>(w, x, gs_ptr, y, *k_dim_p, *rows_p, m, xs);
}
// the shared-X body: grid (ceil(row_tiles / 4), ceil(M / MT)), block 256, MT = 16 TBK = 64 / 128 tokens; dynamic LDS = two X tiles
#define CROW_GEMM_PIPE_ENTRY(NAME, TBK, OCC)                                                                                   \
    extern "C" __global__ void __launch_bounds__(256, OCC) NAME(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x, \
                                                           const float* __restrict__ gs_ptr, float* __restrict__ y,            \
                                                           const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,    \
                                                           const int* __restrict__ m_p) {                                      \
        /* 256 threads; X is addressed with 32-bit element offsets */                                                         \
        if (block_threads() != 256 || *m_p < 1 || (unsigned long long)*m_p * (unsigned long long)*k_dim_p > 0xffffffffull) {   \
            if (threadIdx.x == 0) atomicOr(crow::g_ws.status, crow::STATUS_BAD_SHAPE);                                         \
            return;                                                                                                            \
        }                                                                                                                      \
        crow::gemm_pipe_body<TBK>(w, x, gs_ptr, y, *k_dim_p, *rows_p, *m_p, (__bf16*)crow_dyn_lds);                            \
    }
CROW_GEMM_PIPE_ENTRY(gemm_nvfp4_bf16_m48, 3, 2)
CROW_GEMM_PIPE_ENTRY(gemm_nvfp4_bf16_m64, 4, 2)
CROW_GEMM_PIPE_ENTRY(gemm_nvfp4_bf16_m96, 6, 1)
CROW_GEMM_PIPE_ENTRY(gemm_nvfp4_bf16, 8, 1)
// the wide shared-X body: grid (ceil(row_tiles / 8), ceil(M / MT)), block 512, MT = 16 TBK tokens; dynamic LDS = two X tiles
#define CROW_GEMM_WIDE_ENTRY(NAME, TBK)                                                                                        \
    extern "C" __global__ void __launch_bounds__(512, 1) NAME(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x, \
                                                         const float* __restrict__ gs_ptr, float* __restrict__ y,              \
                                                         const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,      \
                                                         const int* __restrict__ m_p) {                                        \
        /* 512 threads; X is addressed with 32-bit element offsets */                                                         \
        if (block_threads() != 512 || *m_p < 1 || (unsigned long long)*m_p * (unsigned long long)*k_dim_p > 0xffffffffull) {   \
            if (threadIdx.x == 0) atomicOr(crow::g_ws.status, crow::STATUS_BAD_SHAPE);                                         \
            return;                                                                                                            \
        }                                                                                                                      \
        crow::gemm_wide_body<TBK>(w, x, gs_ptr, y, *k_dim_p, *rows_p, *m_p, (__bf16*)crow_dyn_lds);                            \
    }
CROW_GEMM_WIDE_ENTRY(gemm_nvfp4_bf16_w48, 3)
CROW_GEMM_WIDE_ENTRY(gemm_nvfp4_bf16_w64, 4)
CROW_GEMM_WIDE_ENTRY(gemm_nvfp4_bf16_w80, 5)
CROW_GEMM_WIDE_ENTRY(gemm_nvfp4_bf16_w96, 6)

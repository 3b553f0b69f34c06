// NVFP4 GEMV family for gfx950: y[m][row] = gs * sum_k W[row][k] * x[m][k], M <= 4 activation rows.
//
// Mapping.  One wavefront owns one 64-row x 256-column tile at a time and multiplies it on the matrix
// cores: v_mfma_f32_16x16x32_bf16 with the WEIGHT rows on the N side (16 rows per instruction), 32
// columns on the K side and the activation rows on the M side.  The weights are read exactly once,
// as 16-byte-per-lane non-temporal loads that cover 1024 contiguous bytes per instruction, and every
// dword a lane loads is its B operand as it stands (layout.h): eight E2M1 codes become eight exact
// bf16 values with four v_cvt_scalef32_pk_bf16_fp4.  The per-16-column UE4M3 scale is NOT multiplied
// into the weights.  Instead the two 16-column halves of a 32-column segment are kept apart on the M
// side - an activation row occupies one operand row that is zero for K >= 16 and another that is zero
// for K < 16 - so that every lane receives, per matrix instruction pair, the unscaled dot product of
// ITS weight row with ONE 16-column sub-block, and applies that sub-block's scale with a single FMA:
//
//   A1 operand rows 0..3 : r-th activation row, columns  0..15 of the segment   (lane group g = 0 of D)
//   A2 operand rows 4..7 : r-th activation row, columns  0..15                  (g = 1)
//   A1 operand rows 8..11: r-th activation row, columns 16..31                  (g = 2)
//   A2 operand rows 12..15: r-th activation row, columns 16..31                 (g = 3)
//   D = A1 * B(row group 2 jp) ; D = A2 * B(row group 2 jp + 1) + D
//   acc[jp][r] = fma(D[r], ue4m3(scale of this lane's row and sub-block), acc[jp][r])
//
// so one FMA per activation row serves two matrix instructions (1024 weights), and the decode costs
// half an instruction per weight.  bf16 activations ride as they are (r = token).  f32 activations are
// split exactly into three bf16 terms (x = hi + mid + lo, 8 + 8 + 8 significant bits by truncation);
// token t's three terms are operand rows 3 t, 3 t + 1, 3 t + 2 (four rows per matrix instruction pair, so M tokens take
// ceil(3 M / 4) pairs per unit pair) and their results are added as (hi + mid) + lo before the scale FMA: every product
// w * term is exact in f32, so the only roundings are the f32 additions, as in any f32 dot product.
//
// Each wave stages its own activation slice (M rows x 256 columns, 512 bytes per bf16 row) in LDS and
// reads its A operands from there with one 16-byte read per lane; lanes whose operand row is zero read
// a zeroed 512-byte area instead.
//
// FP32 accumulation order (per output row and activation row), documented because it differs
// from the reference CPU path's 8-lane order (cpu_nvfp4.rs:22-31) and from its GPU kernel of
// record (kernels_p2.rs:304-347); all three are within the same gamma bound of the exact sum:
//   for each 16-value sub-block: part = the matrix core's f32 sum of the 16 exact products
//       (f32 activations: ((part_hi + part_mid) + part_lo))
//   even and odd sub-blocks of the wave's panels accumulate separately, in column order:
//       acc = fma(part, ue4m3(scale), acc);   then acc_even + acc_odd
//   a row split over S blocks of W waves: unit u = slice * W + wave owns panels u, u + S W, ...;
//   a block adds its waves' sums in wave order, then the blocks' sums are added in slice order
//   y = acc * gs                                               (gs last, as kernels_p2.rs:367)
// The order depends only on (K, slices), never on M or on the row's position: row m of an M-row launch
// is bit-identical to a one-row launch with the same slicing (the verify contract of kernels_p2.rs:391-396).
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
//
// Dynamic LDS of a block (bytes; the launcher sizes it from the block size):
//   [0, 512)                                   zeros
//   [512 + (wave * XR + r) * 560, + 512)       activation staging, XR rows per wave (row stride 560); when a wave has
//                                              finished its panels, the first NR * M * 256 bytes of its area carry its
//                                              partial sums to wave 0 (no separate hand-over area)
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
    // grouped launches: not null = row m of this launch is routed combo c = row_map[m]: it reads activation row
    // c / x_div and writes output row c (strides as above); null = rows 0 .. m - 1 in place
    const int* row_map;
    int x_div;
};

// staging rows per wave: one bf16 row per token, or three (hi, mid, lo) per f32 token, rounded up to whole sets of four
// operand rows (the padding rows are staged as zeros)
template <int M, bool XBF16>
struct XRows {
    static constexpr int value = XBF16 ? M : 4 * ((3 * M + 3) / 4);
};
#define CROW_GEMV_ZERO_BYTES 512
// 512 bytes of data per staged row; the 48 bytes of padding start four consecutive rows 48 bytes apart modulo the 256-byte
// bank cycle, so that the operand reads of a set's rows mostly miss each other (64 bytes would separate them fully:
// measured equal), and twelve rows for each of twelve waves still fit twice into a compute unit's 160 KB
#define CROW_GEMV_XROW_BYTES 560

typedef __attribute__((address_space(3))) unsigned char* lds_p;
__device__ __forceinline__ void lds_store16(lds_p p, unsigned a, unsigned b, unsigned c, unsigned d) {
    *(__attribute__((address_space(3))) u32x4*)p = u32x4{a, b, c, d};
}
__device__ __forceinline__ void lds_store8(lds_p p, unsigned a, unsigned b) { *(__attribute__((address_space(3))) u32x2*)p = u32x2{a, b}; }

// 8 codes (one dword) -> 8 exact bf16 values: a matrix-instruction operand
__device__ __forceinline__ bf16x8 decode8(unsigned codes) {
    u32x4 r;
    r.x = __builtin_bit_cast(unsigned, fp4x2_to_bf16<0>(codes));
    r.y = __builtin_bit_cast(unsigned, fp4x2_to_bf16<1>(codes));
    r.z = __builtin_bit_cast(unsigned, fp4x2_to_bf16<2>(codes));
    r.w = __builtin_bit_cast(unsigned, fp4x2_to_bf16<3>(codes));
    return __builtin_bit_cast(bf16x8, r);
}

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

// The activation slice of one panel, fetched into registers (before the weight loads are issued, so that its
// data does not queue behind them) and then written to the wave's LDS rows.
template <int M, bool XBF16>
struct XStage;
template <int M>
struct XStage<M, true> {
    uint4 v[(M + 1) / 2];
    __device__ __forceinline__ void fetch(const void* x, const size_t (&xoff)[M], int col0, int k_dim, int m_rows, int lane) {
        const int c = lane & 31, col = col0 + 8 * c;
#pragma unroll
        for (int t0 = 0; t0 < M; t0 += 2) {
            const int tok = t0 + (lane >> 5);
            v[t0 / 2] = make_uint4(0, 0, 0, 0);
            // rows in place: offset = row * stride (xoff[1] is the stride then); gathered rows: one of two uniform offsets
            const size_t o0 = xoff[t0], o1 = xoff[t0 + 1 < M ? t0 + 1 : t0];
            if (tok < m_rows && col < k_dim) v[t0 / 2] = *(const uint4*)((const unsigned short*)x + ((lane >> 5) ? o1 : o0) + col);
        }
    }
    __device__ __forceinline__ void store(lds_p xw, int lane) const {
#pragma unroll
        for (int t0 = 0; t0 < M; t0 += 2) {
            const int tok = t0 + (lane >> 5);
            if (tok < M) lds_store16(xw + tok * CROW_GEMV_XROW_BYTES + 16 * (lane & 31), v[t0 / 2].x, v[t0 / 2].y, v[t0 / 2].z, v[t0 / 2].w);
        }
    }
};
template <int M>
struct XStage<M, false> {
    float4 v[M];
    __device__ __forceinline__ void fetch(const void* x, const size_t (&xoff)[M], int col0, int k_dim, int m_rows, int lane) {
        const int col = col0 + 4 * lane;
#pragma unroll
        for (int t = 0; t < M; t++) {
            v[t] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (t < m_rows && col < k_dim) v[t] = *(const float4*)((const float*)x + xoff[t] + col);
        }
    }
    // x = hi + mid + lo exactly: each term keeps the next 8 significant bits (truncation; the subtractions are exact)
    __device__ __forceinline__ static void split(float f, unsigned& hi, unsigned& mid, unsigned& lo) {
        hi = __float_as_uint(f) & 0xffff0000u;
        const float r1 = __fsub_rn(f, __uint_as_float(hi));
        mid = __float_as_uint(r1) & 0xffff0000u;
        const float r2 = __fsub_rn(r1, __uint_as_float(mid));
        lo = __float_as_uint(r2) & 0xffff0000u;
    }
    __device__ __forceinline__ void store(lds_p xw, int lane) const {
#pragma unroll
        for (int t = 0; t < M; t++) {
            unsigned h[4], m[4], l[4];
            split(v[t].x, h[0], m[0], l[0]);
            split(v[t].y, h[1], m[1], l[1]);
            split(v[t].z, h[2], m[2], l[2]);
            split(v[t].w, h[3], m[3], l[3]);
            // bf16 pairs: high halves of (odd element, even element)
            lds_p row = xw + (3 * t) * CROW_GEMV_XROW_BYTES + 8 * lane;
            lds_store8(row, __builtin_amdgcn_perm(h[1], h[0], 0x07060302u), __builtin_amdgcn_perm(h[3], h[2], 0x07060302u));
            lds_store8(row + CROW_GEMV_XROW_BYTES, __builtin_amdgcn_perm(m[1], m[0], 0x07060302u), __builtin_amdgcn_perm(m[3], m[2], 0x07060302u));
            lds_store8(row + 2 * CROW_GEMV_XROW_BYTES, __builtin_amdgcn_perm(l[1], l[0], 0x07060302u), __builtin_amdgcn_perm(l[3], l[2], 0x07060302u));
        }
#pragma unroll
        for (int r = 3 * M; r < XRows<M, false>::value; r++) lds_store8(xw + r * CROW_GEMV_XROW_BYTES + 8 * lane, 0u, 0u);
    }
};

// One 32-column segment S of a panel: 4 * NR units.  `a1`, `a2` are this lane's LDS addresses of its A1 / A2 operand
// for segment 0 of set q (or of the zero area); `acc[r][jp][m]` as described at the top of the file.
template <int NR, int M, bool XBF16, int S>
struct Segment {
    // f32: the 3 M split rows (token t: rows 3 t, 3 t + 1, 3 t + 2 = hi, mid, lo) fill sets of four operand rows in order
    static constexpr int NSET = XBF16 ? 1 : (3 * M + 3) / 4;
    // `a1`, `a2`: this lane's LDS address of its A1 / A2 operand of segment 0, set 0; set q is `step` bytes further
    // (0 for a lane that reads the zero area)
    __device__ __forceinline__ static void run(const uint4 (&sc)[NR], const uint4 (&cd)[NR][CROW_STEPS], lds_p a1, lds_p a2, int step1,
                                               int step2, float (&acc)[NR][2][M]) {
        typedef __attribute__((address_space(3))) const u32x4* lds_v4;
        bf16x8 A1[NSET], A2[NSET];
#pragma unroll
        for (int q = 0; q < NSET; q++) {
            A1[q] = __builtin_bit_cast(bf16x8, *(lds_v4)(a1 + q * step1 + 64 * S));
            A2[q] = __builtin_bit_cast(bf16x8, *(lds_v4)(a2 + q * step2 + 64 * S));
        }
#pragma unroll
        for (int jp = 0; jp < 2; jp++) {
#pragma unroll
            for (int r = 0; r < NR; r++) {
                const bf16x8 B0 = decode8(u4_get(cd[r][S], 2 * jp)), B1 = decode8(u4_get(cd[r][S], 2 * jp + 1));
                const float sv = e4m3_to_f32<S & 3>(u4_get(sc[r], 2 * jp + (S >> 2)));
                f32x4 D[NSET];
#pragma unroll
                for (int q = 0; q < NSET; q++) {
                    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
                    D[q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A1[q], B0, z, 0, 0, 0);
                    D[q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A2[q], B1, D[q], 0, 0, 0);
                }
#pragma unroll
                for (int m = 0; m < M; m++) {
                    if (XBF16) {
                        acc[r][jp][m] = __builtin_fmaf(D[0][m], sv, acc[r][jp][m]);
                    } else {
                        const float hi = D[(3 * m) / 4][(3 * m) % 4], mid = D[(3 * m + 1) / 4][(3 * m + 1) % 4], lo = D[(3 * m + 2) / 4][(3 * m + 2) % 4];
                        acc[r][jp][m] = __builtin_fmaf(__fadd_rn(__fadd_rn(hi, mid), lo), sv, acc[r][jp][m]);
                    }
                }
            }
        }
    }
};

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

// The cross-block hand-over for any per-lane vector of NV partial sums (all of them live): the protocol the GEMV body uses,
// for callers outside it.  Returns true in the block that arrived last, with `v` = the sum over slices in slice order;
// false in every other block (which must not touch the output).  Wave-uniform control flow; call from one wave.
template <int NV>
__device__ __forceinline__ bool slice_hand_over(float (&v)[NV], unsigned tile_id, int slice, int slices, const Workspace& ws, int lane) {
    const size_t need = ((size_t)tile_id + 1) * slices * NV * 64;
    if (need > ws.partial_floats || tile_id >= ws.counter_slots) {
        if (lane == 0) atomicOr(ws.status, STATUS_WORKSPACE_TOO_SMALL);
        return false;
    }
    typedef __attribute__((address_space(1))) float* gf_p;
    typedef __attribute__((address_space(1))) unsigned* gu_p;
    gf_p base = (gf_p)ws.partials + (size_t)tile_id * slices * NV * 64;
    gf_p mine = base + (size_t)slice * NV * 64;
    gu_p counter = (gu_p)ws.counters + tile_id;
#pragma unroll
    for (int i = 0; i < NV; i++) __hip_atomic_store(mine + i * 64 + lane, v[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    device_order();
    unsigned arrived = 0;
    if (lane == 0) arrived = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    if (arrived != (unsigned)slices - 1) return false;
    device_order();
#pragma unroll
    for (int i = 0; i < NV; i++) v[i] = 0.0f;
    constexpr int PB = NV >= 32 ? 1 : (NV >= 16 ? 2 : 4);
    for (int s0 = 0; s0 < slices; s0 += PB) {
        float t[PB][NV];
#pragma unroll
        for (int j = 0; j < PB; j++)
#pragma unroll
            for (int i = 0; i < NV; i++)
                t[j][i] = s0 + j < slices ? __hip_atomic_load(base + ((size_t)(s0 + j) * NV + i) * 64 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.0f;
#pragma unroll
        for (int j = 0; j < PB; j++)
            if (s0 + j < slices) {
#pragma unroll
                for (int i = 0; i < NV; i++) v[i] += t[j][i];
            }
    }
    if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

// out[r][m] in lane l = the wave's partial dot product of tile row l (of tensor r) with activation row m, summed
// over panels p = p0, p0 + stride, ...  `xw` is the wave's own staging area, `zero` the block's zeroed 512 bytes.
template <int NR, int M, bool XBF16>
__device__ __forceinline__ void tile_accumulate(const unsigned char* const (&w)[2], int rt, int panels, int p0, int stride, int k_dim,
                                                const void* x, const size_t (&xoff)[M], int m_rows, lds_p xw, lds_p zero, float (&out)[NR][M]) {
    constexpr int NSET = XBF16 ? 1 : (3 * M + 3) / 4;
    constexpr int SET_ROWS = XBF16 ? M : 4;  // live operand rows of a set (f32: padding rows are staged as zeros)
    // register-hungry instantiations keep the segments apart: the next segment's operands are not fetched early
    constexpr bool LEAN = NR * NSET >= 2 && !XBF16;
    const int lane = lane_id();
    // this lane as a holder of A operand row i = lane % 16, K group g = lane / 16 (K indices 8 g .. 8 g + 7)
    const int g = lane >> 4, i = lane & 15, r4 = i & 3;
    const bool live = ((g >> 1) == (i >> 3)) && r4 < SET_ROWS;  // the row's 16-column half is this K group's half
    const bool second = ((i >> 2) & 1) != 0;                    // rows 4..7, 12..15 belong to A2
    lds_p data = xw + r4 * CROW_GEMV_XROW_BYTES + 16 * g;
    const lds_p a1 = (live && !second) ? data : zero + 16 * g, a2 = (live && second) ? data : zero + 16 * g;
    const int step1 = (live && !second) ? SET_ROWS * CROW_GEMV_XROW_BYTES : 0, step2 = (live && second) ? SET_ROWS * CROW_GEMV_XROW_BYTES : 0;
    float acc[NR][2][M];
#pragma unroll
    for (int r = 0; r < NR; r++)
#pragma unroll
        for (int jp = 0; jp < 2; jp++)
#pragma unroll
            for (int m = 0; m < M; m++) acc[r][jp][m] = 0.0f;
    for (int p = p0; p < panels; p += stride) {
        XStage<M, XBF16> xs;
        xs.fetch(x, xoff, p * CROW_PANEL_COLS, k_dim, m_rows, lane);
        uint4 sc[NR], cd[NR][CROW_STEPS];
        load_tile<NR>(w, rt, panels, p, lane, sc, cd);
        xs.store(xw, lane);
        __builtin_amdgcn_wave_barrier();  // the reads below follow the writes above in program order (same wave)
        Segment<NR, M, XBF16, 0>::run(sc, cd, a1, a2, step1, step2, acc);
        if (LEAN) __builtin_amdgcn_sched_barrier(0);
        Segment<NR, M, XBF16, 1>::run(sc, cd, a1, a2, step1, step2, acc);
        if (LEAN) __builtin_amdgcn_sched_barrier(0);
        Segment<NR, M, XBF16, 2>::run(sc, cd, a1, a2, step1, step2, acc);
        if (LEAN) __builtin_amdgcn_sched_barrier(0);
        Segment<NR, M, XBF16, 3>::run(sc, cd, a1, a2, step1, step2, acc);
        if (LEAN) __builtin_amdgcn_sched_barrier(0);
        Segment<NR, M, XBF16, 4>::run(sc, cd, a1, a2, step1, step2, acc);
        if (LEAN) __builtin_amdgcn_sched_barrier(0);
        Segment<NR, M, XBF16, 5>::run(sc, cd, a1, a2, step1, step2, acc);
        if (LEAN) __builtin_amdgcn_sched_barrier(0);
        Segment<NR, M, XBF16, 6>::run(sc, cd, a1, a2, step1, step2, acc);
        if (LEAN) __builtin_amdgcn_sched_barrier(0);
        Segment<NR, M, XBF16, 7>::run(sc, cd, a1, a2, step1, step2, acc);
        if (LEAN) __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_wave_barrier();  // ... and the next panel's writes follow these reads
    }
    // lane (g, n) holds row 16 (2 jp + (g & 1)) + n, sub-block parity g >> 1.  Even + odd sub-blocks (lanes l and l + 32),
    // then rows 0..31 (jp = 0) stay in lanes 0..31 and rows 32..63 (jp = 1) move to lanes 32..63: lane = tile row.
#pragma unroll
    for (int r = 0; r < NR; r++)
#pragma unroll
        for (int m = 0; m < M; m++) {
            float v[2];
#pragma unroll
            for (int jp = 0; jp < 2; jp++) {
                const unsigned a = __float_as_uint(acc[r][jp][m]);
                const u32x2 sw = __builtin_amdgcn_permlane32_swap(a, a, false, false);  // .x = lanes 0..31 everywhere, .y = 32..63
                v[jp] = __fadd_rn(__uint_as_float(sw.x), __uint_as_float(sw.y));
            }
            out[r][m] = lane < 32 ? v[0] : v[1];
        }
}

typedef __attribute__((address_space(1))) float* gfloat_p;
typedef __attribute__((address_space(1))) unsigned* guint_p;
typedef __attribute__((address_space(1))) int* gint_p;

// The body every GEMV entry point runs.  The caller has already offset the pointers in `a` for
// its token group / combo `z`, which only indexes the workspace here.  `lds` is the block's dynamic
// LDS, laid out as described at the top of the file for XR_ALLOC staging rows per wave.
template <int NR, int M, bool XBF16, int EPI, int XR_ALLOC, bool THIN = false>
__device__ __forceinline__ void gemv_body(const GemvArgs& a, unsigned z, lds_p lds, const Workspace& ws) {
    static_assert(XRows<M, XBF16>::value <= XR_ALLOC, "staging rows");
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), waves = block_threads() >> 6;  // wave-uniform on purpose
    const int slice = (int)blockIdx.x, slices = (int)gridDim.x;
    const int rt = (int)blockIdx.y;
    const int row_tiles = (int)gridDim.y;
    const int panels = (a.k_dim + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS;
    const int m_rows = a.m < M ? a.m : M;
    const unsigned tile_id = z * (unsigned)row_tiles + (unsigned)rt;
    // element offsets of this launch's activation and output rows
    size_t xoff[M], yoff[M];
#pragma unroll
    for (int m = 0; m < M; m++) {
        if (a.row_map != nullptr) {
            const int c = a.row_map[m < m_rows ? m : 0];
            xoff[m] = (size_t)(c / a.x_div) * a.x_stride;
            yoff[m] = (size_t)c * a.y_stride;
        } else {
            xoff[m] = (size_t)m * a.x_stride;
            yoff[m] = (size_t)m * a.y_stride;
        }
    }

    if (rt * CROW_TILE_ROWS >= a.rows) return;  // a grid taller than the tensor: the whole block (and every slice of the tile) leaves
    if constexpr (THIN && NR == 2) {
        if (waves & 1) {  // the two tensors take half of the block's waves each (uniform over the block: nobody waits at a barrier)
            if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
            return;
        }
    }
    lds_p zero = lds;
    lds_p xw = lds + CROW_GEMV_ZERO_BYTES + wave * (XR_ALLOC * CROW_GEMV_XROW_BYTES);
    // a wave's partial sums for wave 0 go where its staged activations were (dead by then): area w, NR * M rows of 256 bytes
    typedef __attribute__((address_space(3))) float* lds_f;
    static_assert(NR * M * 256 <= XR_ALLOC * CROW_GEMV_XROW_BYTES, "hand-over rows fit the staging area");
    auto red_of = [&](int w) -> lds_f { return (lds_f)(lds + CROW_GEMV_ZERO_BYTES + w * (XR_ALLOC * CROW_GEMV_XROW_BYTES)); };
    if (threadIdx.x < CROW_GEMV_ZERO_BYTES / 16) lds_store16(zero + 16 * threadIdx.x, 0, 0, 0, 0);
    if (waves > 1) __syncthreads();
    else __builtin_amdgcn_wave_barrier();

    float acc[NR][M];
    if constexpr (THIN && NR == 2) {
        // One tile per wave: the block runs 2 W waves, waves 0 .. W - 1 take the panels of tensor 0 and waves W .. 2 W - 1 the
        // same panels of tensor 1.  This keeps the register count (and so the number of resident waves) of the
        // one-tensor kernel; the arithmetic per row is that of the two-tiles-per-wave form.
        const int wpt = waves >> 1;               // waves per tensor (W)
        const int r_own = wave >= wpt ? 1 : 0;    // wave-uniform
        const int pw = wave - r_own * wpt;
        float part[1][M];
        const unsigned char* const w_own[2] = {r_own != 0 ? a.w[1] : a.w[0], nullptr};  // a select, never an indexed read
        tile_accumulate<1, M, XBF16>(w_own, rt, panels, slice * wpt + pw, slices * wpt, a.k_dim, a.x, xoff, m_rows, xw, zero, part);
        // waves of the block -> wave 0, per tensor in wave order
#pragma unroll
        for (int m = 0; m < M; m++) acc[0][m] = part[0][m];
        if (wave > 0) {
            lds_f mine = red_of(wave);
#pragma unroll
            for (int m = 0; m < M; m++)
                if (m < m_rows) mine[m * 64 + lane] = part[0][m];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int w = 1; w < wpt; w++) {
#pragma unroll
            for (int m = 0; m < M; m++)
                if (m < m_rows) acc[0][m] += red_of(w)[m * 64 + lane];
        }
#pragma unroll
        for (int m = 0; m < M; m++) acc[1][m] = m < m_rows ? red_of(wpt)[m * 64 + lane] : 0.0f;
        for (int w = wpt + 1; w < waves; w++) {
#pragma unroll
            for (int m = 0; m < M; m++)
                if (m < m_rows) acc[1][m] += red_of(w)[m * 64 + lane];
        }
    } else {
        tile_accumulate<NR, M, XBF16>(a.w, rt, panels, slice * waves + wave, slices * waves, a.k_dim, a.x, xoff, m_rows, xw, zero, acc);
        // waves of the block -> wave 0, in wave order
        if (waves > 1) {
            if (wave > 0) {
                lds_f mine = red_of(wave);
#pragma unroll
                for (int r = 0; r < NR; r++)
#pragma unroll
                    for (int m = 0; m < M; m++)
                        if (m < m_rows) mine[(r * M + m) * 64 + lane] = acc[r][m];
            }
            __syncthreads();
            if (wave > 0) return;
            for (int w = 1; w < waves; w++) {
#pragma unroll
                for (int r = 0; r < NR; r++)
#pragma unroll
                    for (int m = 0; m < M; m++)
                        if (m < m_rows) acc[r][m] += red_of(w)[(r * M + m) * 64 + lane];
            }
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
            if (m < m_rows) a.y[yoff[m] + row] = acc[0][m] * gs;
    } else {
        const float gg = a.gs[0][0], gu = a.gs[NR - 1][0];
#pragma unroll
        for (int m = 0; m < M; m++)
            if (m < m_rows) a.y[yoff[m] + row] = silu_mul(acc[0][m] * gg, acc[NR - 1][m] * gu);
    }
}

}  // namespace crow

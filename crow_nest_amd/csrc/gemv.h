// NVFP4 GEMV family for gfx950: y[m][row] = gs * sum_k W[row][k] * x[m][k], M <= 4 activation rows.
//
// Mapping.  A workgroup owns one 16-row STRIP of the tensor (layout.h) and, for K up to 16384, ALL of its columns: wave w of
// the block walks a run of consecutive 256-column groups, four of them (9 KB) in flight at any time, and the block's waves
// meet in LDS.  Nothing crosses workgroups, so there is no workspace, no arrival counter and no device-scope ordering on this path.
// Only tensors whose strip does not fit one block's waves (K > 16384, e.g. the 17408-column down projection) are cut into S
// column slices whose blocks hand their 16 sums over through the library workspace (slice_hand_over below).
// The weights are read exactly once, as non-temporal loads that cover 1024 contiguous bytes per instruction, issued
// before anything else: their addresses depend only on the kernel arguments and on K / 64, which the launcher passes BY VALUE
// (`pairs`), never on a word behind a pointer - the first weight load leaves one scalar round trip after the wave starts.
//
// Arithmetic.  v_mfma_f32_16x16x32_bf16 with the 16 WEIGHT rows on the N side, 32 columns on the K side and the activation rows
// on the M side.  Every dword a lane loads is its B operand as it stands: eight E2M1 codes become eight exact bf16 values with
// four v_cvt_scalef32_pk_bf16_fp4.  The per-16-column UE4M3 scale is NOT multiplied into the weights.  Instead the four
// sub-blocks of a 64-column pair are kept apart on the M side - an activation row occupies one operand row that is zero for
// K >= 16 and another that is zero for K < 16, in each of the pair's two instructions - so that every lane receives, per pair,
// the unscaled dot product of ITS weight row with ONE 16-column sub-block, and applies that sub-block's scale with a single FMA:
//
//   A1 operand rows 0..3 : r-th activation row, columns  0..15 of segment 0 of the pair   (lane group g = 0 of D)
//   A2 operand rows 4..7 : r-th activation row, columns  0..15 of segment 1               (g = 1)
//   A1 operand rows 8..11: r-th activation row, columns 16..31 of segment 0               (g = 2)
//   A2 operand rows 12..15: r-th activation row, columns 16..31 of segment 1              (g = 3)
//   D = A1 * B(segment 0) ; D = A2 * B(segment 1) + D
//   acc[r] = fma(D[r], ue4m3(scale of this lane's row and sub-block), acc[r])
//
// so one FMA per activation row serves two matrix instructions (1024 weights), and the decode costs half an instruction per
// weight.  bf16 activations ride as they are (r = token).  f32 activations are split exactly into three bf16 terms
// (x = hi + mid + lo, 8 + 8 + 8 significant bits by truncation); token t's three terms are operand rows 3 t, 3 t + 1, 3 t + 2
// (four rows per instruction pair, so M tokens take ceil(3 M / 4) instruction pairs per weight pair) and their results are
// added as (hi + mid) + lo before the scale FMA: every product w * term is exact in f32, so the only roundings are the f32
// additions, as in any f32 dot product.
//
// Each wave stages its own activation slice in LDS, group by group (bf16 rows, 512 bytes per group, two groups deep), while
// its weight loads are in flight, and reads its A operands from there with one 16-byte read per lane; lanes whose operand
// row is zero read a zeroed area instead.
//
// FP32 accumulation order (per output row and activation row), documented because it differs from the reference CPU path's
// 8-lane order (cpu_nvfp4.rs:22-31) and from its GPU kernel of record (kernels_p2.rs:304-347); all three are within the same
// gamma bound of the exact sum:
//   for each 16-value sub-block: part = the matrix core's f32 sum of the 16 exact products
//       (f32 activations: ((part_hi + part_mid) + part_lo))
//   the four sub-block classes c = 0..3 of a pair (columns 16 c .. 16 c + 15) accumulate separately over the wave's pairs, in
//       column order: acc_c = fma(part, ue4m3(scale), acc_c);  then (acc_0 + acc_1) + (acc_2 + acc_3)
//   the block adds its waves' sums in wave order (= column order); a row split over S blocks adds the blocks' sums in slice order
//   y = acc * gs                                               (gs last, as kernels_p2.rs:367)
// The order depends only on (K, waves, slices), never on M or on the row's position: row m of an M-row launch is bit-identical
// to a one-row launch with the same geometry (the verify contract of kernels_p2.rs:391-396).
//
// Launch geometry: grid (strips, S, Z), block 64 * W * NR threads (NR = 2 for the fused gate / up kernels: waves 0 .. W - 1 take
// tensor 0 and waves W .. 2 W - 1 the same columns of tensor 1).  blockIdx.x = strip, blockIdx.y = column slice, blockIdx.z =
// token group / expert combo.  The strip's G groups are dealt to the S * W units in runs of floor(G / (S W)) or one more;
// unit u = slice * W + wave.
//
// Dynamic LDS of a block (bytes; the launcher sizes it from the block size):
//   [0, 640)                        zeros
//   [640 + wave * 2 * XR * 560, ..) the wave's activation staging: two slots of XR rows of 560 bytes; when a wave has finished
//                                   its groups, the first 64 M bytes of its area carry its 16 M sums to wave 0
#pragma once
#include "device_common.h"

namespace crow {

enum Epilogue { EPI_SCALE = 0, EPI_SILU_GU = 1 };

// Measurement builds only (-DCROW_TRACE): per-block timestamps (the 100 MHz wall clock) of the phases of a launch, read back
// with crow_hip_trace_read.  Slot 0 = the block's first instruction, 1 = its first waves past their first requests and the
// block barrier, 2 = the last wave done with its groups, 3 = the stores issued.
#ifdef CROW_TRACE
__device__ unsigned long long crow_trace[16384 * 8];
#define CROW_STAMP(slot) do { if (threadIdx.x == 0 && blockIdx.y == 0 && blockIdx.x < 16384) crow_trace[blockIdx.x * 8 + (slot)] = wall_clock64(); } while (0)
#define CROW_STAMP_LAST(slot) do { if ((threadIdx.x & 63) == 0 && blockIdx.y == 0 && blockIdx.x < 16384) atomicMax(&crow_trace[blockIdx.x * 8 + (slot)], (unsigned long long)wall_clock64()); } while (0)
#else
#define CROW_STAMP(slot) do { } while (0)
#define CROW_STAMP_LAST(slot) do { } while (0)
#endif

struct GemvArgs {
    const unsigned char* w[2];  // tiled tensors (w[1] only for EPI_SILU_GU: the `up` matrix)
    const float* gs[2];
    const void* x;       // [M][x_stride] f32 (or bf16 when XBF16)
    size_t x_stride;     // elements between activation rows
    float* y;            // [..][y_stride]
    size_t y_stride;     // elements between output rows; 0 = the row count (*rows_p), which is then only needed at the store
    int pairs;           // K / 64, by value from the launcher
    const int* k_dim_p;  // the caller's K word: only compared with `pairs` before anything is stored
    const int* rows_p;   // the row count: read for the stores only
    // output row of activation row m: y_row0 + m, or - grouped launches, row_map not null - the routed combo
    // c = row_map[m], which reads activation row c / x_div and writes output row c
    int y_row0 = 0;
    const int* row_map = nullptr;
    int x_div = 1;
    int* argmax_out = nullptr;      // not null: also leave this strip's greedy-argmax candidate of y row 0 (fused lm_head head)
    // a launch whose row count came by value: the word it must agree with, checked before anything is stored
    const int* count_p = nullptr;
    int count_expect = 0;
};
__device__ __forceinline__ GemvArgs gemv_args(const unsigned char* w0, const unsigned char* w1, const float* gs0, const float* gs1, const void* x,
                                              size_t x_stride, float* y, size_t y_stride, int pairs, const int* k_dim_p, const int* rows_p) {
    GemvArgs a;
    a.w[0] = w0, a.w[1] = w1, a.gs[0] = gs0, a.gs[1] = gs1, a.x = x, a.x_stride = x_stride, a.y = y, a.y_stride = y_stride;
    a.pairs = pairs, a.k_dim_p = k_dim_p, a.rows_p = rows_p;
    return a;
}

// A wave keeps this many 256-column groups (2304 bytes each) in flight: a ring of register slots that is refilled group by
// group as the wave walks along its strip.
#define CROW_GEMV_RING 4
// One staged activation row of one group: 512 bytes of bf16 values.  The 48 bytes of padding start four consecutive rows
// 48 bytes apart modulo the 128-byte bank cycle, so that the operand reads of a set's rows miss each other.
#define CROW_GEMV_XROW_BYTES 560
#define CROW_GEMV_ZERO_BYTES 640  // a zeroed row (512 bytes + what a zero lane's reads reach past the last pair's offset)

// The staging a wave needs for M activation rows: XR rows per group (one bf16 row per token, or three - hi, mid, lo - per f32
// token), two groups deep (the next group is staged while the current one is multiplied).
template <int M, bool XBF16>
struct Staging {
    static constexpr int XR = XBF16 ? M : 3 * M;
    static constexpr int SLOT = XR * CROW_GEMV_XROW_BYTES;
    static constexpr int PER_WAVE = 2 * SLOT;  // also carries the wave's 16 M sums to wave 0 afterwards (>= 256 bytes)
};
// the dynamic LDS of a block: the zero area, then one staging area per wave, sized for the widest body of the entry point
CROW_HD static constexpr int crow_gemv_lds_per_wave(int mmax, bool xbf16) { return 2 * (xbf16 ? mmax : 3 * mmax) * CROW_GEMV_XROW_BYTES; }

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

// x = hi + mid + lo exactly: each term keeps the next 8 significant bits (truncation; the subtractions are exact)
__device__ __forceinline__ void split3(float f, unsigned& hi, unsigned& mid, unsigned& lo) {
    hi = __float_as_uint(f) & 0xffff0000u;
    const float r1 = __fsub_rn(f, __uint_as_float(hi));
    mid = __float_as_uint(r1) & 0xffff0000u;
    const float r2 = __fsub_rn(r1, __uint_as_float(mid));
    lo = __float_as_uint(r2) & 0xffff0000u;
}

// One 256-column group of NS strips: four pairs.  `a1[q]`, `a2[q]` are this lane's LDS addresses of its A1 / A2 operand for pair
// 0 of the group's staging slot, set q (or of the zero area).  The activation operands of a pair are read once and serve all
// NS strips; per strip the operation sequence is that of a one-strip walk.
template <int M, bool XBF16, int NS>
__device__ __forceinline__ void group_multiply(const unsigned (&sc)[NS], const u32x4 (&cd)[NS][2], const lds_p (&a1)[XBF16 ? 1 : (3 * M + 3) / 4],
                                               const lds_p (&a2)[XBF16 ? 1 : (3 * M + 3) / 4], float (&acc)[NS][M]) {
    constexpr int NSET = XBF16 ? 1 : (3 * M + 3) / 4;
    typedef __attribute__((address_space(3))) const u32x4* lds_v4;
#pragma unroll
    for (int jj = 0; jj < CROW_GROUP_PAIRS; jj++) {
        bf16x8 A1[NSET], A2[NSET];
#pragma unroll
        for (int q = 0; q < NSET; q++) {
            A1[q] = __builtin_bit_cast(bf16x8, *(lds_v4)(a1[q] + 128 * jj));
            A2[q] = __builtin_bit_cast(bf16x8, *(lds_v4)(a2[q] + 128 * jj));
        }
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const u32x4 c = cd[s][jj >> 1];
            const bf16x8 B0 = decode8((jj & 1) ? c.z : c.x), B1 = decode8((jj & 1) ? c.w : c.y);
            const float sv = jj == 0 ? e4m3_to_f32<0>(sc[s]) : (jj == 1 ? e4m3_to_f32<1>(sc[s]) : (jj == 2 ? e4m3_to_f32<2>(sc[s]) : e4m3_to_f32<3>(sc[s])));
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
                    acc[s][m] = __builtin_fmaf(D[0][m], sv, acc[s][m]);
                } else {
                    const float hi = D[(3 * m) / 4][(3 * m) % 4], mid = D[(3 * m + 1) / 4][(3 * m + 1) % 4], lo = D[(3 * m + 2) / 4][(3 * m + 2) % 4];
                    acc[s][m] = __builtin_fmaf(__fadd_rn(__fadd_rn(hi, mid), lo), sv, acc[s][m]);
                }
            }
        }
    }
}

// A wave's walk along its strip: groups first .. first + count - 1, RING of them in flight at any time.
//
//   issue<J>(g)    requests group g into ring slot J: its activations (4 columns per lane and token; every lane always loads -
//                  a lane whose columns lie beyond K reads the row's last four instead and drops them when staging - so no load
//                  sits behind a branch and the compiler can count the loads in flight exactly) and its 2304 weight bytes
//   stage<J>(g)    writes slot J's activations as bf16 rows into LDS staging slot J % 2
//   multiply<J>()  four pairs of matrix instructions on slot J against LDS slot J % 2
//
// Steady state, per group: stage the NEXT group (its activations were requested right behind the current group's weights, so
// they are here once those are), multiply the current one, refill its slot with the group RING further on.  Everything is
// unrolled by RING so that every register index, LDS offset and wait count is static; the walk ends in one of RING tails, chosen
// by how many groups are left to request.
template <int M, bool XBF16>
struct StripWalk {
    typedef Staging<M, XBF16> St;
    static constexpr int NSET = XBF16 ? 1 : (3 * M + 3) / 4;
    typedef typename std::conditional<XBF16, u32x2, f32x4>::type XV;  // plain vector types: they live in registers
    unsigned sc[CROW_GEMV_RING][1];
    u32x4 cd[CROW_GEMV_RING][1][2];
    XV xv[CROW_GEMV_RING][M];
    lds_p a1[2][NSET], a2[2][NSET];  // this lane's operand addresses in the two staging slots (or in the zero area)
    lds_p xw;
    const unsigned char* wl;  // the lane's view of the wave's first group
    const unsigned char* xl;  // the lane's view of the wave's first column of activation row 0
    size_t xoff[M];           // byte offsets of the activation rows
    int col_lane, k_dim, lane;
    float acc[1][M];

    __device__ __forceinline__ void init(const unsigned char* strip, int first, int k_dim_, const void* x, const size_t (&xoff_elems)[M], lds_p xw_,
                                         lds_p zero) {
        lane = lane_id();
        xw = xw_;
        k_dim = k_dim_;
        wl = strip + (size_t)first * CROW_GROUP_BYTES;
        col_lane = first * CROW_GROUP_COLS + 4 * lane;
        xl = (const unsigned char*)x;
#pragma unroll
        for (int m = 0; m < M; m++) {
            xoff[m] = xoff_elems[m] * (XBF16 ? 2 : 4);
            acc[0][m] = 0.0f;
        }
        // this lane as a holder of A operand row i = lane % 16, K group g = lane / 16 (K indices 8 g .. 8 g + 7)
        const int g = lane >> 4, i = lane & 15, r4 = i & 3;
        const bool half_ok = (g >> 1) == (i >> 3);      // the row's 16-column half is this K group's half
        const bool second = ((i >> 2) & 1) != 0;        // rows 4..7, 12..15 belong to A2 (segment 1 of the pair: 64 bytes on)
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
            for (int q = 0; q < NSET; q++) {
                const int row = 4 * q + r4;
                const bool live = half_ok && row < St::XR;
                lds_p data = xw + s * St::SLOT + row * CROW_GEMV_XROW_BYTES + 16 * g;
                a1[s][q] = (live && !second) ? data : zero + 16 * g;
                a2[s][q] = (live && second) ? data + 64 : zero + 16 * g;
            }
    }
    // activations of group g into x slot J (g % RING == J)
    template <int J>
    __device__ __forceinline__ void issue_x(int g) {
        const int col = col_lane + g * CROW_GROUP_COLS;
        const size_t o = (size_t)(col < k_dim ? col : k_dim - 4) * (XBF16 ? 2 : 4);
#pragma unroll
        for (int t = 0; t < M; t++) xv[J][t] = *(const __attribute__((address_space(1))) XV*)(xl + xoff[t] + o);
    }
    // weights of group g into slot J
    template <int J>
    __device__ __forceinline__ void issue_w(int g) {
        const unsigned char* p = wl + (size_t)g * CROW_GROUP_BYTES;
        sc[J][0] = stream_load_u32((const unsigned*)p + lane);
        cd[J][0][0] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES) + lane);
        cd[J][0][1] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES + 1024) + lane);
    }
    template <int J>
    __device__ __forceinline__ void stage(int g) {
        const bool in = col_lane + g * CROW_GROUP_COLS < k_dim;
        lds_p slot = xw + (J & 1) * St::SLOT + 8 * lane;
#pragma unroll
        for (int t = 0; t < M; t++) {
            if constexpr (XBF16) {
                lds_store8(slot + t * CROW_GEMV_XROW_BYTES, in ? xv[J][t].x : 0u, in ? xv[J][t].y : 0u);
            } else {
                unsigned h[4], m[4], l[4];
                split3(in ? xv[J][t].x : 0.f, h[0], m[0], l[0]);
                split3(in ? xv[J][t].y : 0.f, h[1], m[1], l[1]);
                split3(in ? xv[J][t].z : 0.f, h[2], m[2], l[2]);
                split3(in ? xv[J][t].w : 0.f, h[3], m[3], l[3]);
                // bf16 pairs: high halves of (odd element, even element)
                lds_p row = slot + (3 * t) * CROW_GEMV_XROW_BYTES;
                lds_store8(row, __builtin_amdgcn_perm(h[1], h[0], 0x07060302u), __builtin_amdgcn_perm(h[3], h[2], 0x07060302u));
                lds_store8(row + CROW_GEMV_XROW_BYTES, __builtin_amdgcn_perm(m[1], m[0], 0x07060302u), __builtin_amdgcn_perm(m[3], m[2], 0x07060302u));
                lds_store8(row + 2 * CROW_GEMV_XROW_BYTES, __builtin_amdgcn_perm(l[1], l[0], 0x07060302u), __builtin_amdgcn_perm(l[3], l[2], 0x07060302u));
            }
        }
        __builtin_amdgcn_wave_barrier();  // (the wave's LDS accesses execute in order: this only keeps the compiler from reordering them)
    }
    template <int J>
    __device__ __forceinline__ void multiply() {
        group_multiply<M, XBF16, 1>(sc[J], cd[J], a1[J & 1], a2[J & 1], acc);
        __builtin_amdgcn_wave_barrier();
        // a group is one scheduling region: without the fence the scheduler pulls the decodes of several groups forward in the
        // long straight-line tails of the walk and runs out of registers there
        __builtin_amdgcn_sched_barrier(0);
    }

    // groups g .. g + N - 1 (N <= RING) are requested into slots 0 .. N - 1 - activations first, so that they do not queue
    // behind the weights
    template <int N>
    __device__ __forceinline__ void start(int g) {
        if (N > 0) issue_x<0>(g);
        if (N > 1) issue_x<1>(g + 1);
        if (N > 2) issue_x<2>(g + 2);
        if (N > 3) issue_x<3>(g + 3);
        if (N > 0) issue_w<0>(g);
        if (N > 1) issue_w<1>(g + 1);
        if (N > 2) issue_w<2>(g + 2);
        if (N > 3) issue_w<3>(g + 3);
    }
    // On entry: the weights of groups g0 .. g0 + 3 are in (or on their way to) slots 0..3, group g0 is staged, the activations of
    // g0 + 1 .. g0 + 4 are in (or on their way to) their x slots.  The quad multiplies its four groups and, if REFILL, requests
    // the weights of the next four into the slots it frees.  The activations of groups g0 + 5 .. g0 + 8 are requested in any case,
    // each as soon as its x slot has been staged: a request for a group beyond the wave's run reads columns that exist (or the
    // row's last four) and is never used.  On return group g0 + 4 is staged if REFILL.
    template <bool REFILL>
    __device__ __forceinline__ void quad(int g0) {
        stage<1>(g0 + 1);
        issue_x<1>(g0 + 5);
        multiply<0>();
        if (REFILL) issue_w<0>(g0 + 4);
        stage<2>(g0 + 2);
        issue_x<2>(g0 + 6);
        multiply<1>();
        if (REFILL) issue_w<1>(g0 + 5);
        stage<3>(g0 + 3);
        issue_x<3>(g0 + 7);
        multiply<2>();
        if (REFILL) issue_w<2>(g0 + 6);
        if (REFILL) {
            stage<0>(g0 + 4);
            issue_x<0>(g0 + 8);
        }
        multiply<3>();
        if (REFILL) issue_w<3>(g0 + 7);
    }
    // the last N < RING groups g0 .. g0 + N - 1 sit in slots 0 .. N - 1, group g0 is staged
    template <int N>
    __device__ __forceinline__ void rest(int g0) {
        if (N > 1) stage<1>(g0 + 1);
        if (N > 0) multiply<0>();
        if (N > 2) stage<2>(g0 + 2);
        if (N > 1) multiply<1>();
        if (N > 2) multiply<2>();
    }
    template <int N>
    __device__ __forceinline__ void remainder(int g) {
        start<N>(g);
        stage<0>(g);
        rest<N>(g);
    }
    // The whole walk over `count` groups: the full quads as a pipeline (every quad's loads in flight while the one before is
    // multiplied), then what is left (count % 4 groups) on its own.  `mid` is whatever the block has to do between a wave's
    // first requests and its first use of LDS (zeroing the zero area, a block barrier): it runs once, after the first loads
    // have left.  Paths with different loads in flight never meet before a wait that matters, so the waits count exactly.
    template <class Mid>
    __device__ __forceinline__ void go(int count, Mid mid) {
        const int nq = count >> 2, r = count & 3;
        if (nq > 0) {
            start<4>(0);
            mid();
            stage<0>(0);
            issue_x<0>(4);
            // (one copy of each body, and no branch whose two sides begin alike: the compiler hoists what two successors of a
            // branch have in common, here every decode of the ring, above the branch - and runs out of registers there)
            int q = 0;
            for (; q + 1 < nq; q++) quad<true>(4 * q);
            quad<false>(4 * q);
            if (r == 3) remainder<3>(4 * nq);
            else if (r == 2) remainder<2>(4 * nq);
            else if (r == 1) remainder<1>(4 * nq);
        } else if (r == 3) {
            start<3>(0);
            mid();
            stage<0>(0);
            rest<3>(0);
        } else if (r == 2) {
            start<2>(0);
            mid();
            stage<0>(0);
            rest<2>(0);
        } else if (r == 1) {
            start<1>(0);
            mid();
            stage<0>(0);
            rest<1>(0);
        } else {
            mid();
        }
    }
    // out[m] in every lane l = the wave's partial dot product of strip row l % 16 with activation row m.
    // lane (g, n) holds sub-block class 2 (g & 1) + (g >> 1) of row n: classes (0 + 1) + (2 + 3) = (g0 + g2) + (g1 + g3)
    __device__ __forceinline__ void finish(float (&out)[M]) const {
#pragma unroll
        for (int m = 0; m < M; m++) {
            const unsigned a = __float_as_uint(acc[0][m]);
            const u32x2 sw = __builtin_amdgcn_permlane32_swap(a, a, false, false);  // .x = lanes 0..31's value, .y = lanes 32..63's
            const unsigned b = __float_as_uint(__fadd_rn(__uint_as_float(sw.x), __uint_as_float(sw.y)));
            const u32x2 sq = __builtin_amdgcn_permlane16_swap(b, b, false, false);  // .x = the even 16-lane group's value, .y = the odd one's
            out[m] = __fadd_rn(__uint_as_float(sq.x), __uint_as_float(sq.y));
        }
    }
};

// StripWalk for bf16 activations with the activation traffic halved: a lane asks for 8 columns (16 bytes) of a PAIR of groups
// at once - lanes 0..31 cover the pair's first group, lanes 32..63 its second - and one 16-byte LDS store per row stages both
// groups' rows (the staged bytes, the operand reads and every sum are StripWalk's: same bits).  Per group that is 3.5 vector
// memory instructions instead of 4 and half an LDS store instead of one.  The activation rows must be 16-byte aligned.
#ifndef CROW_BF16_XPAIRS
#define CROW_BF16_XPAIRS 1
#endif
template <int M>
struct StripWalkPairs {
    typedef Staging<M, true> St;
    unsigned sc[CROW_GEMV_RING][1];
    u32x4 cd[CROW_GEMV_RING][1][2];
    u32x4 xp[2][M];           // pair slot P holds groups 4 q + 2 P, 4 q + 2 P + 1
    lds_p a1[2][1], a2[2][1];
    lds_p xw;
    const unsigned char* wl;
    const unsigned char* xl;
    size_t xoff[M];
    int col_lane, k_dim, lane;
    float acc[1][M];

    __device__ __forceinline__ void init(const unsigned char* strip, int first, int k_dim_, const void* x, const size_t (&xoff_elems)[M], lds_p xw_,
                                         lds_p zero) {
        lane = lane_id();
        xw = xw_;
        k_dim = k_dim_;
        wl = strip + (size_t)first * CROW_GROUP_BYTES;
        col_lane = first * CROW_GROUP_COLS + 8 * lane;
        xl = (const unsigned char*)x;
#pragma unroll
        for (int m = 0; m < M; m++) {
            xoff[m] = xoff_elems[m] * 2;
            acc[0][m] = 0.0f;
        }
        const int g = lane >> 4, i = lane & 15, r4 = i & 3;
        const bool half_ok = (g >> 1) == (i >> 3);
        const bool second = ((i >> 2) & 1) != 0;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            const bool live = half_ok && r4 < St::XR;
            lds_p data = xw + s * St::SLOT + r4 * CROW_GEMV_XROW_BYTES + 16 * g;
            a1[s][0] = (live && !second) ? data : zero + 16 * g;
            a2[s][0] = (live && second) ? data + 64 : zero + 16 * g;
        }
    }
    // activations of groups g, g + 1 (g even in the wave's own count) into pair slot P
    template <int P>
    __device__ __forceinline__ void issue_xp(int g) {
        const int col = col_lane + g * CROW_GROUP_COLS;
        const size_t o = (size_t)(col < k_dim ? col : k_dim - 8) * 2;
#pragma unroll
        for (int t = 0; t < M; t++) xp[P][t] = *(const __attribute__((address_space(1))) u32x4*)(xl + xoff[t] + o);
    }
    template <int J>
    __device__ __forceinline__ void issue_w(int g) {
        const unsigned char* p = wl + (size_t)g * CROW_GROUP_BYTES;
        sc[J][0] = stream_load_u32((const unsigned*)p + lane);
        cd[J][0][0] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES) + lane);
        cd[J][0][1] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES + 1024) + lane);
    }
    // pair slot P -> the two LDS staging slots (group g into slot 0, group g + 1 into slot 1)
    template <int P>
    __device__ __forceinline__ void stage_pair(int g) {
        const bool in = col_lane + g * CROW_GROUP_COLS < k_dim;
        lds_p dst = xw + (lane >> 5) * St::SLOT + 16 * (lane & 31);
#pragma unroll
        for (int t = 0; t < M; t++)
            lds_store16(dst + t * CROW_GEMV_XROW_BYTES, in ? xp[P][t].x : 0u, in ? xp[P][t].y : 0u, in ? xp[P][t].z : 0u, in ? xp[P][t].w : 0u);
        __builtin_amdgcn_wave_barrier();
    }
    template <int J>
    __device__ __forceinline__ void multiply() {
        group_multiply<M, true, 1>(sc[J], cd[J], a1[J & 1], a2[J & 1], acc);
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    template <int N>
    __device__ __forceinline__ void start(int g) {
        if (N > 0) issue_xp<0>(g);
        if (N > 2) issue_xp<1>(g + 2);
        if (N > 0) issue_w<0>(g);
        if (N > 1) issue_w<1>(g + 1);
        if (N > 2) issue_w<2>(g + 2);
        if (N > 3) issue_w<3>(g + 3);
    }
    // On entry: the weights of g0 .. g0 + 3 are in (or on their way to) slots 0..3, the pair (g0, g0 + 1) is staged, pair slot 1
    // holds (or awaits) g0 + 2, g0 + 3 and pair slot 0 g0 + 4, g0 + 5.  Requests beyond the wave's run read columns that exist
    // (or the row's last eight) and are never used.  On return the pair (g0 + 4, g0 + 5) is staged if REFILL.
    template <bool REFILL>
    __device__ __forceinline__ void quad(int g0) {
        multiply<0>();
        if (REFILL) issue_w<0>(g0 + 4);
        multiply<1>();
        if (REFILL) issue_w<1>(g0 + 5);
        stage_pair<1>(g0 + 2);
        issue_xp<1>(g0 + 6);
        multiply<2>();
        if (REFILL) issue_w<2>(g0 + 6);
        multiply<3>();
        if (REFILL) {
            issue_w<3>(g0 + 7);
            stage_pair<0>(g0 + 4);
            issue_xp<0>(g0 + 8);
        }
    }
    template <int N>
    __device__ __forceinline__ void rest(int g0) {
        if (N > 0) multiply<0>();
        if (N > 1) multiply<1>();
        if (N > 2) {
            stage_pair<1>(g0 + 2);
            multiply<2>();
        }
    }
    template <int N>
    __device__ __forceinline__ void remainder(int g) {
        start<N>(g);
        stage_pair<0>(g);
        rest<N>(g);
    }
    template <class Mid>
    __device__ __forceinline__ void go(int count, Mid mid) {
        const int nq = count >> 2, r = count & 3;
        if (nq > 0) {
            start<4>(0);
            mid();
            stage_pair<0>(0);
            issue_xp<0>(4);
            int q = 0;
            for (; q + 1 < nq; q++) quad<true>(4 * q);
            quad<false>(4 * q);
            if (r == 3) remainder<3>(4 * nq);
            else if (r == 2) remainder<2>(4 * nq);
            else if (r == 1) remainder<1>(4 * nq);
        } else if (r == 3) {
            start<3>(0);
            mid();
            stage_pair<0>(0);
            rest<3>(0);
        } else if (r == 2) {
            start<2>(0);
            mid();
            stage_pair<0>(0);
            rest<2>(0);
        } else if (r == 1) {
            start<1>(0);
            mid();
            stage_pair<0>(0);
            rest<1>(0);
        } else {
            mid();
        }
    }
    __device__ __forceinline__ void finish(float (&out)[M]) const {
#pragma unroll
        for (int m = 0; m < M; m++) {
            const unsigned a = __float_as_uint(acc[0][m]);
            const u32x2 sw = __builtin_amdgcn_permlane32_swap(a, a, false, false);
            const unsigned b = __float_as_uint(__fadd_rn(__uint_as_float(sw.x), __uint_as_float(sw.y)));
            const u32x2 sq = __builtin_amdgcn_permlane16_swap(b, b, false, false);
            out[m] = __fadd_rn(__uint_as_float(sq.x), __uint_as_float(sq.y));
        }
    }
};

// The walk of a wave that takes NS adjacent strips at once (the kernels for several activation rows): per group the staged
// activations and the operand reads from LDS serve NS x 16 weight rows, which is what bounds those kernels - at four f32 rows a
// group's operand reads are ten times its weight bytes.  Two groups (NS x 2304 bytes each) in flight; per strip and
// activation row the operation sequence is StripWalk's, so the sums are the same bits.
//   wl[s]   the lane's view of the wave's first group of strip s (a strip beyond the tensor: any strip that exists; its
//           sums are never stored)
template <int M, bool XBF16, int NS>
struct MultiWalk {
    typedef Staging<M, XBF16> St;
    static constexpr int NSET = XBF16 ? 1 : (3 * M + 3) / 4;
    typedef typename std::conditional<XBF16, u32x2, f32x4>::type XV;
    unsigned sc[2][NS];
    u32x4 cd[2][NS][2];
    XV xv[2][M];
    lds_p a1[2][NSET], a2[2][NSET];
    lds_p xw;
    const unsigned char* wl[NS];
    const unsigned char* xl;
    size_t xoff[M];
    int col_lane, k_dim, lane;
    float acc[NS][M];

    __device__ __forceinline__ void init(const unsigned char* const (&strip)[NS], int first, int k_dim_, const void* x, const size_t (&xoff_elems)[M],
                                         lds_p xw_, lds_p zero) {
        lane = lane_id();
        xw = xw_;
        k_dim = k_dim_;
#pragma unroll
        for (int s = 0; s < NS; s++) wl[s] = strip[s] + (size_t)first * CROW_GROUP_BYTES;
        col_lane = first * CROW_GROUP_COLS + 4 * lane;
        xl = (const unsigned char*)x;
#pragma unroll
        for (int m = 0; m < M; m++) {
            xoff[m] = xoff_elems[m] * (XBF16 ? 2 : 4);
#pragma unroll
            for (int s = 0; s < NS; s++) acc[s][m] = 0.0f;
        }
        const int g = lane >> 4, i = lane & 15, r4 = i & 3;
        const bool half_ok = (g >> 1) == (i >> 3);
        const bool second = ((i >> 2) & 1) != 0;
#pragma unroll
        for (int sl = 0; sl < 2; sl++)
#pragma unroll
            for (int q = 0; q < NSET; q++) {
                const int row = 4 * q + r4;
                const bool live = half_ok && row < St::XR;
                lds_p data = xw + sl * St::SLOT + row * CROW_GEMV_XROW_BYTES + 16 * g;
                a1[sl][q] = (live && !second) ? data : zero + 16 * g;
                a2[sl][q] = (live && second) ? data + 64 : zero + 16 * g;
            }
    }
    template <int J>
    __device__ __forceinline__ void issue_x(int g) {
        const int col = col_lane + g * CROW_GROUP_COLS;
        const size_t o = (size_t)(col < k_dim ? col : k_dim - 4) * (XBF16 ? 2 : 4);
#pragma unroll
        for (int t = 0; t < M; t++) xv[J][t] = *(const __attribute__((address_space(1))) XV*)(xl + xoff[t] + o);
    }
    template <int J>
    __device__ __forceinline__ void issue_w(int g) {
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const unsigned char* p = wl[s] + (size_t)g * CROW_GROUP_BYTES;
            sc[J][s] = stream_load_u32((const unsigned*)p + lane);
            cd[J][s][0] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES) + lane);
            cd[J][s][1] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES + 1024) + lane);
        }
    }
    template <int J>
    __device__ __forceinline__ void stage(int g) {
        const bool in = col_lane + g * CROW_GROUP_COLS < k_dim;
        lds_p slot = xw + J * St::SLOT + 8 * lane;
#pragma unroll
        for (int t = 0; t < M; t++) {
            if constexpr (XBF16) {
                lds_store8(slot + t * CROW_GEMV_XROW_BYTES, in ? xv[J][t].x : 0u, in ? xv[J][t].y : 0u);
            } else {
                unsigned h[4], m[4], l[4];
                split3(in ? xv[J][t].x : 0.f, h[0], m[0], l[0]);
                split3(in ? xv[J][t].y : 0.f, h[1], m[1], l[1]);
                split3(in ? xv[J][t].z : 0.f, h[2], m[2], l[2]);
                split3(in ? xv[J][t].w : 0.f, h[3], m[3], l[3]);
                lds_p row = slot + (3 * t) * CROW_GEMV_XROW_BYTES;
                lds_store8(row, __builtin_amdgcn_perm(h[1], h[0], 0x07060302u), __builtin_amdgcn_perm(h[3], h[2], 0x07060302u));
                lds_store8(row + CROW_GEMV_XROW_BYTES, __builtin_amdgcn_perm(m[1], m[0], 0x07060302u), __builtin_amdgcn_perm(m[3], m[2], 0x07060302u));
                lds_store8(row + 2 * CROW_GEMV_XROW_BYTES, __builtin_amdgcn_perm(l[1], l[0], 0x07060302u), __builtin_amdgcn_perm(l[3], l[2], 0x07060302u));
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
    template <int J>
    __device__ __forceinline__ void multiply() {
        group_multiply<M, XBF16, NS>(sc[J], cd[J], a1[J], a2[J], acc);
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    // On entry: the weights of groups g0, g0 + 1 are in (or on their way to) slots 0, 1; group g0 is staged; the activations of
    // g0 + 1 and g0 + 2 are in (or on their way to) x slots 1 and 0.  Requests for groups beyond the wave's run read columns
    // that exist (or the row's last four) and are never used.  On return, if REFILL, the same holds for g0 + 2.
    template <bool REFILL>
    __device__ __forceinline__ void duo(int g0) {
        stage<1>(g0 + 1);
        issue_x<1>(g0 + 3);
        multiply<0>();
        if (REFILL) {
            issue_w<0>(g0 + 2);
            stage<0>(g0 + 2);
            issue_x<0>(g0 + 4);
        }
        multiply<1>();
        if (REFILL) issue_w<1>(g0 + 3);
    }
    // (one copy of each body, and no branch whose two sides begin alike: see StripWalk::go)
    template <class Mid>
    __device__ __forceinline__ void go(int count, Mid mid) {
        const int even = count & ~1;
        if (even > 0) {
            issue_x<0>(0);
            issue_x<1>(1);
            issue_w<0>(0);
            issue_w<1>(1);
            mid();
            stage<0>(0);
            issue_x<0>(2);
            int g = 0;
            for (; g + 2 < even; g += 2) duo<true>(g);
            duo<false>(g);
            if (count & 1) {
                issue_x<0>(even);
                issue_w<0>(even);
                stage<0>(even);
                multiply<0>();
            }
        } else if (count == 1) {
            issue_x<0>(0);
            issue_w<0>(0);
            mid();
            stage<0>(0);
            multiply<0>();
        } else {
            mid();
        }
    }
    __device__ __forceinline__ void finish(float (&out)[NS][M]) const {
#pragma unroll
        for (int s = 0; s < NS; s++)
#pragma unroll
            for (int m = 0; m < M; m++) {
                const unsigned a = __float_as_uint(acc[s][m]);
                const u32x2 sw = __builtin_amdgcn_permlane32_swap(a, a, false, false);
                const unsigned b = __float_as_uint(__fadd_rn(__uint_as_float(sw.x), __uint_as_float(sw.y)));
                const u32x2 sq = __builtin_amdgcn_permlane16_swap(b, b, false, false);
                out[s][m] = __fadd_rn(__uint_as_float(sq.x), __uint_as_float(sq.y));
            }
    }
};

// The walk of a wave over MANY strips of FEW groups (short K: the routed experts' slabs, K = 2048 / 512 -> eight / two groups
// per strip).  Walking such strips one block each means tens of thousands of blocks that each stage the same activation rows,
// fill a pipeline of a few groups and drain it again.  Here the block stages the tile's activation rows ONCE (all groups of all
// M rows; they never change along the walk) and every wave streams a run of consecutive strips - whose groups are one
// contiguous run of 2304-byte records in memory - through the ring of four, with no activation traffic, no staging and no
// register slots for activations inside the loop.  NR = 2: a strip of `gate` is followed by the same strip of `up` (the
// tensor `up_off` bytes further on) and the two sums leave together.  A strip is walked by this one wave from its first group
// to its last, which is the operation sequence of StripWalk for a strip that one wave walks alone: the same bits.
template <int M, int NR>
struct TileWalk {
    static constexpr int XR = 3 * M, NSET = (3 * M + 3) / 4, SLOT = XR * CROW_GEMV_XROW_BYTES;
    unsigned sc[CROW_GEMV_RING][1];
    u32x4 cd[CROW_GEMV_RING][1][2];
    lds_p a1b[NSET], a2b[NSET];  // this lane's operand addresses in group 0's staged rows (or in the zero area) ...
    int st1[NSET], st2[NSET];    // ... and what a group further on adds to them (0 for the zero area)
    // the request side: the next record, its group and its tensor; the multiply side: the same for the next record to multiply
    const unsigned char* p_next;
    ptrdiff_t up_off;
    int groups, gi_req, t_req, gi, t_mul, done, lane;
    float first_sum;
    float acc[1][M];

    // f32 activations of one group of one row -> three bf16 rows (hi, mid, lo) of the group's staged area; a lane = 4 columns
    static __device__ __forceinline__ void stage_row(lds_p staged, int g, int t, f32x4 v, int lane_) {
        unsigned h[4], m[4], l[4];
        split3(v.x, h[0], m[0], l[0]);
        split3(v.y, h[1], m[1], l[1]);
        split3(v.z, h[2], m[2], l[2]);
        split3(v.w, h[3], m[3], l[3]);
        lds_p row = staged + g * SLOT + (3 * t) * CROW_GEMV_XROW_BYTES + 8 * lane_;
        lds_store8(row, __builtin_amdgcn_perm(h[1], h[0], 0x07060302u), __builtin_amdgcn_perm(h[3], h[2], 0x07060302u));
        lds_store8(row + CROW_GEMV_XROW_BYTES, __builtin_amdgcn_perm(m[1], m[0], 0x07060302u), __builtin_amdgcn_perm(m[3], m[2], 0x07060302u));
        lds_store8(row + 2 * CROW_GEMV_XROW_BYTES, __builtin_amdgcn_perm(l[1], l[0], 0x07060302u), __builtin_amdgcn_perm(l[3], l[2], 0x07060302u));
    }
    __device__ __forceinline__ void init(const unsigned char* first_record, ptrdiff_t up_off_, int groups_, lds_p staged, lds_p zero) {
        lane = lane_id();
        p_next = first_record;
        up_off = up_off_;
        groups = groups_;
        gi_req = 0, t_req = 0, gi = 0, t_mul = 0, done = 0, first_sum = 0.0f;
#pragma unroll
        for (int m = 0; m < M; m++) acc[0][m] = 0.0f;
        // (the operand addressing of StripWalk::init, one staged area per group)
        const int g = lane >> 4, i = lane & 15, r4 = i & 3;
        const bool half_ok = (g >> 1) == (i >> 3);
        const bool second = ((i >> 2) & 1) != 0;
#pragma unroll
        for (int q = 0; q < NSET; q++) {
            const int row = 4 * q + r4;
            const bool live = half_ok && row < XR;
            lds_p data = staged + row * CROW_GEMV_XROW_BYTES + 16 * g;
            a1b[q] = (live && !second) ? data : zero + 16 * g;
            st1[q] = (live && !second) ? SLOT : 0;
            a2b[q] = (live && second) ? data + 64 : zero + 16 * g;
            st2[q] = (live && second) ? SLOT : 0;
        }
    }
    // requests the wave's next record into slot J
    template <int J>
    __device__ __forceinline__ void issue_w() {
        const unsigned char* p = p_next;
        sc[J][0] = stream_load_u32((const unsigned*)p + lane);
        cd[J][0][0] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES) + lane);
        cd[J][0][1] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES + 1024) + lane);
        p_next += CROW_GROUP_BYTES;
        if (++gi_req == groups) {  // wave-uniform
            gi_req = 0;
            if (NR == 2) {  // gate strip s -> up strip s -> gate strip s + 1
                p_next += t_req == 0 ? up_off - (ptrdiff_t)groups * CROW_GROUP_BYTES : -up_off;
                t_req ^= 1;
            }
        }
    }
    // the next record sits in slot J: multiply it by its group's staged rows; behind a strip's last group the strip's sums are
    // closed, and behind the last tensor's `emit(strips finished before, first, last)` - in lane l the dot products of strip
    // row l % 16 with activation row l / 16, of the first tensor and of the last (one tensor: `last` only)
    template <int J, class Emit>
    __device__ __forceinline__ void multiply(Emit& emit) {
        lds_p a1[NSET], a2[NSET];
#pragma unroll
        for (int q = 0; q < NSET; q++) {
            a1[q] = a1b[q] + gi * st1[q];
            a2[q] = a2b[q] + gi * st2[q];
        }
        group_multiply<M, false, 1>(sc[J], cd[J], a1, a2, acc);
        __builtin_amdgcn_sched_barrier(0);
        if (++gi == groups) {  // wave-uniform
            gi = 0;
            float v = 0.0f;
#pragma unroll
            for (int m = 0; m < M; m++) {  // (StripWalk::finish)
                const unsigned a = __float_as_uint(acc[0][m]);
                const u32x2 sw = __builtin_amdgcn_permlane32_swap(a, a, false, false);
                const unsigned b = __float_as_uint(__fadd_rn(__uint_as_float(sw.x), __uint_as_float(sw.y)));
                const u32x2 sq = __builtin_amdgcn_permlane16_swap(b, b, false, false);
                const float o = __fadd_rn(__uint_as_float(sq.x), __uint_as_float(sq.y));
                v = (lane >> 4) == m ? o : v;
                acc[0][m] = 0.0f;
            }
            if (NR == 2 && t_mul == 0) {
                first_sum = v;
                t_mul = 1;
            } else {
                emit(done, first_sum, v);
                done++;
                t_mul = 0;
            }
        }
    }
    // `count` records (whole strips of every tensor) from the wave's first one; `mid` runs once, after the first loads have
    // left: the block's staging and its barrier
    template <class Mid, class Emit>
    __device__ __forceinline__ void go(int count, Mid mid, Emit emit) {
        const int nq = count >> 2, r = count & 3;
        if (nq > 0) {
            issue_w<0>();
            issue_w<1>();
            issue_w<2>();
            issue_w<3>();
            mid();
            for (int q = 0; q + 1 < nq; q++) {
                multiply<0>(emit);
                issue_w<0>();
                multiply<1>(emit);
                issue_w<1>();
                multiply<2>(emit);
                issue_w<2>();
                multiply<3>(emit);
                issue_w<3>();
            }
            multiply<0>(emit);
            if (r > 0) issue_w<0>();
            multiply<1>(emit);
            if (r > 1) issue_w<1>();
            multiply<2>(emit);
            if (r > 2) issue_w<2>();
            multiply<3>(emit);
            if (r > 0) multiply<0>(emit);
            if (r > 1) multiply<1>(emit);
            if (r > 2) multiply<2>(emit);
        } else {
            if (r > 0) issue_w<0>();
            if (r > 1) issue_w<1>();
            if (r > 2) issue_w<2>();
            mid();
            if (r > 0) multiply<0>(emit);
            if (r > 1) multiply<1>(emit);
            if (r > 2) multiply<2>(emit);
        }
    }
};

// Ordering point of the cross-block hand-over.  Every access to the shared partials and counters is an agent-scope atomic:
// the partials are only written by atomic stores and read by atomic loads, which on gfx950 carry the coherence bit that
// makes them bypass the per-die L2 for data other dies may touch; the counters are only touched by read-modify-write
// atomics, which are coherent among themselves.  Never read a counter with a load, atomic or not: it does not see the other
// dies' updates (measured: a polling loop of atomic loads never saw them) - and the compiler turns a read-modify-write with a
// constant identity operand (fetch_add(p, 0)) into exactly such a load.  What is left to guarantee is
// program order between them, which a wait for this wave's outstanding memory operations gives: the partial stores are
// acknowledged before the arrival counter is bumped, and the counter's value is back before any partial is read.  An
// agent-scope fence would add a write-back (release) or an invalidate (acquire) of the whole L2 to exactly this wait;
// neither has anything to do here, because no datum of the hand-over is ever written or read by a plain access, and
// every block paying one was measured at tens of microseconds per launch.
__device__ __forceinline__ void device_order() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("" ::: "memory");
}

// The cross-block hand-over for a per-lane vector of NV partial sums (all of them live).  Returns true in the block that arrived
// last, with `v` = the sum over slices in slice order; false in every other block (which must not touch the output).
// Wave-uniform control flow; call from one wave.
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
    constexpr int PB = NV >= 32 ? 1 : (NV >= 16 ? 2 : (NV >= 4 ? 4 : 8));
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

typedef __attribute__((address_space(3))) float* lds_f;

// The body every GEMV entry point runs.  The caller has already offset the pointers in `a` for its token group / combo `z`,
// which only indexes the workspace here.  `lds` is the block's dynamic LDS, laid out as described at the top of the file and
// sized by the launcher for M_ALLOC rows: entry points that dispatch over M size it for their widest body.
// NS = strips per block: 1 for the one-row kernels (StripWalk); the kernels for several activation rows take NS adjacent strips
// per block, every wave all NS of them over its run of columns (MultiWalk), blockIdx.x = strip / NS.
template <int NR, int M, bool XBF16, int EPI, int M_ALLOC = M, int NS = 1>
__device__ __forceinline__ void gemv_body(const GemvArgs& a, unsigned z, lds_p lds, const Workspace& ws) {
    static_assert(M <= M_ALLOC, "the allocation covers this body");
    constexpr int AREA = crow_gemv_lds_per_wave(M_ALLOC, XBF16);
    static_assert(NS * M * 64 <= AREA, "a wave's sums fit its staging area");
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), waves = block_threads() >> 6;  // wave-uniform on purpose
    CROW_STAMP(0);
    const int strip = (int)blockIdx.x * NS, strips = (int)gridDim.x * NS;
    const int slice = (int)blockIdx.y, slices = (int)gridDim.y;
    const int k_dim = a.pairs * CROW_PAIR_COLS;
    const int groups = (a.pairs + CROW_GROUP_PAIRS - 1) / CROW_GROUP_PAIRS;
    const int wpt = NR == 2 ? waves >> 1 : waves;            // waves per tensor
    const int r_own = (NR == 2 && wave >= wpt) ? 1 : 0;      // wave-uniform
    const int unit = slice * wpt + (wave - r_own * wpt), units = slices * wpt;
    // the strip's groups in runs of floor(groups / units), the first groups % units runs one longer
    const int base = groups / units, rem = groups - base * units;
    // (a two-tensor block launched with an odd number of waves has one wave too many: it takes nothing, and the launch is
    // refused at the store - not here, where the refusal would sit between a wave's start and its first weight load)
    const bool extra_wave = NR == 2 && wave - r_own * wpt >= wpt;
    const int count = extra_wave ? 0 : base + (unit < rem ? 1 : 0), first = unit * base + (unit < rem ? unit : rem);
    const unsigned char* wsel = r_own != 0 ? a.w[1] : a.w[0];  // a select, never an indexed read
    // element offsets of this launch's activation rows, and which output row each of them writes
    size_t xoff[M];
    int yrow[M];
#pragma unroll
    for (int m = 0; m < M; m++) {
        if (a.row_map != nullptr) {
            const int c = a.row_map[m];
            xoff[m] = (size_t)(c / a.x_div) * a.x_stride;
            yrow[m] = c;
        } else {
            xoff[m] = (size_t)m * a.x_stride;
            yrow[m] = a.y_row0 + m;
        }
    }
    lds_p zero = lds;
    lds_p areas = lds + CROW_GEMV_ZERO_BYTES;
    auto mid = [&]() {  // (the wave's first loads have left by now)
        for (int o = 16 * (int)threadIdx.x; o < CROW_GEMV_ZERO_BYTES; o += 16 * (waves << 6)) lds_store16(zero + o, 0, 0, 0, 0);
        if (waves > 1) __syncthreads();
        else __builtin_amdgcn_wave_barrier();
        CROW_STAMP(1);
    };
    float part[NS][M];
    if constexpr (NS == 1) {
        typename std::conditional<XBF16 && CROW_BF16_XPAIRS != 0, StripWalkPairs<M>, StripWalk<M, XBF16>>::type walk;
        walk.init(wsel + (size_t)strip * groups * CROW_GROUP_BYTES, first, k_dim, a.x, xoff, areas + wave * AREA, zero);
        walk.go(count, mid);
        walk.finish(part[0]);
        CROW_STAMP_LAST(2);
    } else {
        // Only the launch's last block can reach past the tensor's last strip: it alone reads the row count before its first
        // weight load, and reads an existing strip instead (the sums of a strip beyond the tensor are never stored).
        int have = NS;
        if (blockIdx.x + 1 == gridDim.x) {
            const int left = (*a.rows_p + CROW_STRIP_ROWS - 1) / CROW_STRIP_ROWS - strip;
            have = left < 1 ? 1 : (left < NS ? left : NS);
        }
        const unsigned char* sp[NS];
#pragma unroll
        for (int s = 0; s < NS; s++) sp[s] = wsel + (size_t)(strip + (s < have ? s : 0)) * groups * CROW_GROUP_BYTES;
        MultiWalk<M, XBF16, NS> walk;
        walk.init(sp, first, k_dim, a.x, xoff, areas + wave * AREA, zero);
        walk.go(count, mid);
        walk.finish(part);
    }

    // waves of the block -> wave 0: lane l of wave 0 takes output (m = l / 16, n = l % 16) of every strip and adds the waves'
    // sums in wave order
    float v[NR * NS];
#pragma unroll
    for (int r = 0; r < NR * NS; r++) v[r] = 0.0f;
    const int mo = lane >> 4, n = lane & 15;
    if (waves > 1) {
        if (lane < 16) {
#pragma unroll
            for (int s = 0; s < NS; s++)
#pragma unroll
                for (int m = 0; m < M; m++) ((lds_f)(areas + wave * AREA))[(s * M + m) * 16 + lane] = part[s][m];
        }
        __syncthreads();
        if (wave > 0) return;
        if (mo < M) {
#pragma unroll
            for (int r = 0; r < NR; r++)
#pragma unroll
                for (int s = 0; s < NS; s++) {
                    v[r * NS + s] = ((lds_f)(areas + (r * wpt) * AREA))[s * M * 16 + lane];
                    for (int w = 1; w < wpt; w++) v[r * NS + s] += ((lds_f)(areas + (r * wpt + w) * AREA))[s * M * 16 + lane];
                }
        }
    } else {
#pragma unroll
        for (int s = 0; s < NS; s++)
#pragma unroll
            for (int m = 0; m < M; m++)
                if (mo == m) v[s] = part[s][m];
    }

    // slices of the block's strips -> the last one to arrive, in slice order
    if (slices > 1 && !slice_hand_over<NR * NS>(v, z * gridDim.x + blockIdx.x, slice, slices, ws, lane)) return;

    const int rows = *a.rows_p;
    // the launch geometry was made for another problem, or the two tensors cannot share the block's waves evenly: nothing is stored
    if (*a.k_dim_p != k_dim || (a.count_p != nullptr && *a.count_p != a.count_expect) || (NR == 2 && (waves & 1)) ||
        (EPI == EPI_SCALE && a.argmax_out != nullptr && (unsigned)strips > ws.head_words)) {
        if (lane == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
        return;
    }
    if constexpr (NS == 1 && EPI == EPI_SCALE) {
        const int row = strip * CROW_STRIP_ROWS + n;
        if (a.argmax_out != nullptr) {
            // fused head: logits out, and this strip's best (value, index) as one ordered key for the finishing kernel that the
            // launcher starts behind this one (misc_kernels.h: argmax_finish).  Same total order as argmax_k.
            const float val = v[0] * a.gs[0][0];
            const bool live = mo == 0 && row < rows;
            if (live) a.y[row] = val;
            const Best b = wave_best(Best{live ? val : -3.0e38f, live ? row : 0});
            if (lane == 0) ws.head[strip] = best_key(b.v, b.i);
            return;
        }
    }
    if (mo >= M) return;
    int yr = yrow[0];
#pragma unroll
    for (int m = 1; m < M; m++)
        if (mo == m) yr = yrow[m];
    const size_t yo = (size_t)yr * (a.y_stride != 0 ? a.y_stride : (size_t)rows);
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const int row = (strip + s) * CROW_STRIP_ROWS + n;
        if (row >= rows) continue;
        if (EPI == EPI_SCALE) {
            a.y[yo + row] = v[s] * a.gs[0][0];
        } else {
            a.y[yo + row] = silu_mul(v[s] * a.gs[0][0], v[(NR - 1) * NS + s] * a.gs[NR - 1][0]);
        }
    }
    CROW_STAMP(3);
}

// The body of a product over strips of few groups (TileWalk): grid.x blocks of W waves, every wave a run of `spw` consecutive
// strips (of each of the NR tensors), all M activation rows staged once per block.  `lds`: the zero area, then one area of
// 3 M staged rows per group.  Strips of at most CROW_TILE_MAX_GROUPS groups.
#define CROW_TILE_MAX_GROUPS 8
template <int M, int NR, int EPI>
__device__ __forceinline__ void tile_body(const GemvArgs& a, int spw, lds_p lds, const Workspace& ws) {
    typedef TileWalk<M, NR> Walk;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), waves = block_threads() >> 6;
    const int k_dim = a.pairs * CROW_PAIR_COLS;
    const int groups = (a.pairs + CROW_GROUP_PAIRS - 1) / CROW_GROUP_PAIRS;
    const int strip0 = ((int)blockIdx.x * waves + wave) * spw;
    size_t xoff[M];
    int yrow[M];
#pragma unroll
    for (int m = 0; m < M; m++) {
        if (a.row_map != nullptr) {
            const int c = a.row_map[m];
            xoff[m] = (size_t)(c / a.x_div) * a.x_stride;
            yrow[m] = c;
        } else {
            xoff[m] = (size_t)m * a.x_stride;
            yrow[m] = a.y_row0 + m;
        }
    }
    // the row count bounds every wave's run (its word arrives with the caller's other words: no round trip of its own), and
    // a grid that does not cover the tensor is refused
    const int strips = (*a.rows_p + CROW_STRIP_ROWS - 1) / CROW_STRIP_ROWS;
    const int left = strips - strip0;
    const int n_strips = left < 0 ? 0 : (left < spw ? left : spw);
    const bool covered = (long long)gridDim.x * waves * spw >= (long long)strips && groups <= CROW_TILE_MAX_GROUPS && spw >= 1;
    lds_p zero = lds, staged = lds + CROW_GEMV_ZERO_BYTES;
    Walk walk;
    walk.init(a.w[0] + (size_t)strip0 * groups * CROW_GROUP_BYTES, NR == 2 ? a.w[1] - a.w[0] : 0, groups, staged, zero);
    int rows = 0;
    float gs0 = 0.0f, gs1 = 0.0f;
    bool ok = true;
    auto mid = [&]() {
        for (int o = 16 * (int)threadIdx.x; o < CROW_GEMV_ZERO_BYTES; o += 16 * (waves << 6)) lds_store16(zero + o, 0, 0, 0, 0);
        // (group, row) pairs dealt to the waves; a lane whose four columns lie beyond K stages zeros
#pragma unroll
        for (int t = 0; t < M; t++)
#pragma unroll
            for (int g = 0; g < CROW_TILE_MAX_GROUPS; g++) {
                if (g >= groups || (t * CROW_TILE_MAX_GROUPS + g) % waves != wave) continue;  // wave-uniform
                const int col = g * CROW_GROUP_COLS + 4 * lane;
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (col < k_dim) v = *(const f32x4*)((const float*)a.x + xoff[t] + col);
                Walk::stage_row(staged, g, t, v, lane);
            }
        rows = *a.rows_p;
        gs0 = a.gs[0][0];
        gs1 = a.gs[NR - 1][0];
        ok = covered && *a.k_dim_p == k_dim && (a.count_p == nullptr || *a.count_p == a.count_expect);
        __syncthreads();
    };
    const int mo = lane >> 4, n = lane & 15;
    int yr = yrow[0];
#pragma unroll
    for (int m = 1; m < M; m++)
        if (mo == m) yr = yrow[m];
    auto emit = [&](int s, float first, float last) {
        const int row = (strip0 + s) * CROW_STRIP_ROWS + n;
        if (ok && mo < M && row < rows) {
            const size_t o = (size_t)yr * (a.y_stride != 0 ? a.y_stride : (size_t)rows) + row;
            if (EPI == EPI_SCALE) a.y[o] = last * gs0;
            else a.y[o] = silu_mul(first * gs0, last * gs1);
        }
    };
    walk.go(covered ? n_strips * NR * groups : 0, mid, emit);
    if (!ok && threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
}

}  // namespace crow

// Kernel entry points of the library.  Names and argument lists follow the reference's kernel
// table (engine/src/kernels.rs:5135-5201, kernels_p2.rs) so that the call sites in
// engine/src/gen.rs keep their `launch_v(k.f(name), ..., &[args])` form; every argument is a
// device address, scalars are 4-byte device words (the reference's own convention,
// engine/src/cuda.rs:1-4).  Where an entry needs one more scalar than its reference twin
// (the row count, which the reference encodes in its grid) it is appended at the END of the
// list and named *_p like the others.
//
// Every entry point of the GEMV family has one more parameter that callers never pass: the geometry word `geo` BY VALUE, which
// the library's launcher takes from the launch dimensions (crow_hip_launch_dims puts it in `gy`) and appends itself: bits 0..19
// = K / 64, bits 20..23 = the activation row count of the launch's LAST token group (0 = not given: read it from memory).  It
// lets a wave address its weights - and fetch its activations - without first waiting for the words behind k_dim_p / m_p to
// arrive from memory; those words are still read, late, and a launch whose values disagree stores nothing.
#pragma once
#include "gemv.h"

using namespace crow;

// The block's dynamic LDS (zeros, activation staging, wave hand-over: gemv.h); the launcher sizes it.
extern __shared__ uint4 crow_dyn_lds[];
#define LDS ((lds_p)crow_dyn_lds)
// After `geo` every entry point of the family takes the descriptor of the scratch memory its launch may use (per-slice partial
// sums, arrival counters, the status word, the argmax key) BY VALUE too: the launcher appends the library's allocation, or -
// crow_hip_launch_noalloc - the one it keeps in a static device array.
//
// First statement of every GEMV entry point: ALL kernel arguments are requested together and waited for once - one scalar
// round trip between the start of a wave and its first weight load.  Left alone the compiler fetches each argument where it
// is first used, behind whatever wait comes before: two or three dependent round trips.
template <typename T>
__device__ __forceinline__ void crow_need_one(T v) {
    asm volatile("" ::"s"(v));
}
__device__ __forceinline__ void crow_need_now() {}
template <typename T, typename... R>
__device__ __forceinline__ void crow_need_now(T v, R... rest) {
    crow_need_one(v);
    crow_need_now(rest...);
}
#define ENTER(...) crow_need_now(ws.status, block_threads(), (int)gridDim.y, __VA_ARGS__)

// ------------------------------------------------------------------ dense GEMV (decode, one row)
// reference: gemv_nvfp4_w, engine/src/kernels_p2.rs:355-368
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_w(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                                const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                const int* __restrict__ k_dim_p, const int* __restrict__ rows_p, int geo, const Workspace ws) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(w, nullptr, gs_ptr, nullptr, x, 0, y, 0, pairs, k_dim_p, rows_p);
    gemv_body<1, 1, false, EPI_SCALE>(a, 0, LDS, ws);
}
// the same product on bf16 activations (exact widening), for models that keep their activations in bf16
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_w_bf16(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                                                     const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                     const int* __restrict__ k_dim_p, const int* __restrict__ rows_p, int geo, const Workspace ws) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(w, nullptr, gs_ptr, nullptr, x, 0, y, 0, pairs, k_dim_p, rows_p);
    gemv_body<1, 1, true, EPI_SCALE>(a, 0, LDS, ws);
}
// reference: gemv_fp4, engine/src/kernels.rs:118-151 (+ rows_p: the reference's grid.x is the row count)
extern "C" __global__ void __launch_bounds__(1024) gemv_fp4(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                            const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                            const int* __restrict__ k_dim_p, const int* __restrict__ rows_p, int geo, const Workspace ws) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(w, nullptr, gs_ptr, nullptr, x, 0, y, 0, pairs, k_dim_p, rows_p);
    gemv_body<1, 1, false, EPI_SCALE>(a, 0, LDS, ws);
}

// lm_head with the greedy argmax fused in: logits[rows] and out_idx[0] = the greedy token from ONE call of the launcher.  Every
// block leaves the best of its 16-row strip as an ordered key in the head's scratch; the launcher starts argmax_finish (one
// block, misc_kernels.h) right behind this kernel, which takes the maximum of ceil(rows / 16) keys instead of re-reading all
// logits.  Replaces lm_head_row + argmax_k (engine/src/gen.rs:4766-4784, engine/src/kernels.rs:4238-4260); same tie rule.
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_w_argmax(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                                       const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                       const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                       int* __restrict__ out_idx, int geo, const Workspace ws) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, out_idx, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(w, nullptr, gs_ptr, nullptr, x, 0, y, 0, pairs, k_dim_p, rows_p);
    a.argmax_out = out_idx;
    gemv_body<1, 1, false, EPI_SCALE>(a, 0, LDS, ws);
}

// ------------------------------------------------------------------ fused gate/up + SiLU (decode)
// reference: gemv_nvfp4_gu, engine/src/kernels_p2.rs:372-389
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_gu(const unsigned char* __restrict__ wg, const unsigned char* __restrict__ wu,
                                                                 const float* __restrict__ x, const float* __restrict__ gs_g,
                                                                 const float* __restrict__ gs_u, float* __restrict__ y,
                                                                 const int* __restrict__ k_dim_p, const int* __restrict__ rows_p, int geo, const Workspace ws) {
    ENTER(wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(wg, wu, gs_g, gs_u, x, 0, y, 0, pairs, k_dim_p, rows_p);
    gemv_body<2, 1, false, EPI_SILU_GU>(a, 0, LDS, ws);
}

// the same on bf16 activations (exact widening)
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_gu_bf16(const unsigned char* __restrict__ wg, const unsigned char* __restrict__ wu,
                                                                      const unsigned short* __restrict__ x, const float* __restrict__ gs_g,
                                                                      const float* __restrict__ gs_u, float* __restrict__ y,
                                                                      const int* __restrict__ k_dim_p, const int* __restrict__ rows_p, int geo, const Workspace ws) {
    ENTER(wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(wg, wu, gs_g, gs_u, x, 0, y, 0, pairs, k_dim_p, rows_p);
    gemv_body<2, 1, true, EPI_SILU_GU>(a, 0, LDS, ws);
}

// ------------------------------------------------------------------ M <= 4 rows (MTP verify)
// Every kernel that multiplies several activation rows at once takes this many adjacent 16-row strips per block (gemv.h:
// MultiWalk); crow_hip_launch_dims sizes grid.x accordingly.
#ifndef CROW_MULTI_STRIPS
#define CROW_MULTI_STRIPS 2
#endif
// ... except the bf16 twins of the verify kernels: their rows ride in one operand set, the operand reads are a sixth of the
// f32 kernels', and one strip per block (the one-row kernels' walk, four groups in flight) measured faster at two rows
#ifndef CROW_MULTI_STRIPS_BF16
#define CROW_MULTI_STRIPS_BF16 1
#endif
template <int NR, bool XBF16, int EPI, int NS = CROW_MULTI_STRIPS>
__device__ __forceinline__ void gemv_m_dispatch(const GemvArgs& a, int m, unsigned z, lds_p lds, const Workspace& ws) {
    if (m < 1 || m > 4) {  // the reference's NVFP4_MMAX (engine/src/kernels_p2.rs:397-400); uniform over the launch
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
        return;
    }
    // one body per M keeps each row's operation sequence identical to the one-row kernel
    switch (m) {
        case 1: gemv_body<NR, 1, XBF16, EPI, 4, NS>(a, z, lds, ws); break;
        case 2: gemv_body<NR, 2, XBF16, EPI, 4, NS>(a, z, lds, ws); break;
        case 3: gemv_body<NR, 3, XBF16, EPI, 4, NS>(a, z, lds, ws); break;
        default: gemv_body<NR, 4, XBF16, EPI, 4, NS>(a, z, lds, ws); break;
    }
}
// The activation row count of a verify launch: from the geometry word when the launcher put it there (then the word behind
// m_p is only compared with it before the store), else read from memory first.
__device__ __forceinline__ int rows_of(GemvArgs& a, int geo, const int* m_p) {
    const int hint = (geo >> 20) & 0xF;
    if (hint == 0) return *m_p;
    a.count_p = m_p;
    a.count_expect = hint;
    return hint;
}
// x [M][k_dim] and y [M][rows] in place: the strides are K (by value) and the row count (needed before the first store only)
// reference: gemv_nvfp4_wm, engine/src/kernels_p2.rs:472-497
extern "C" __global__ void __launch_bounds__(512) gemv_nvfp4_wm(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                                 const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                 const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                 const int* __restrict__ m_p, int geo, const Workspace ws) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, m_p, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(w, nullptr, gs_ptr, nullptr, x, (size_t)pairs * CROW_PAIR_COLS, y, 0, pairs, k_dim_p, rows_p);
    gemv_m_dispatch<1, false, EPI_SCALE>(a, rows_of(a, geo, m_p), 0, LDS, ws);
}
// reference: gemv_nvfp4_gum, engine/src/kernels_p2.rs:499-530
extern "C" __global__ void __launch_bounds__(512) gemv_nvfp4_gum(const unsigned char* __restrict__ wg, const unsigned char* __restrict__ wu,
                                                                   const float* __restrict__ x, const float* __restrict__ gs_g,
                                                                   const float* __restrict__ gs_u, float* __restrict__ y,
                                                                   const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                   const int* __restrict__ m_p, int geo, const Workspace ws) {
    ENTER(wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p, m_p, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(wg, wu, gs_g, gs_u, x, (size_t)pairs * CROW_PAIR_COLS, y, 0, pairs, k_dim_p, rows_p);
    gemv_m_dispatch<2, false, EPI_SILU_GU>(a, rows_of(a, geo, m_p), 0, LDS, ws);
}
// bf16-activation twins of the two verify kernels (X [M][k_dim] bf16, outputs f32)
extern "C" __global__ void __launch_bounds__(512) gemv_nvfp4_wm_bf16(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                                                      const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                      const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                      const int* __restrict__ m_p, int geo, const Workspace ws) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, m_p, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(w, nullptr, gs_ptr, nullptr, x, (size_t)pairs * CROW_PAIR_COLS, y, 0, pairs, k_dim_p, rows_p);
    gemv_m_dispatch<1, true, EPI_SCALE, CROW_MULTI_STRIPS_BF16>(a, rows_of(a, geo, m_p), 0, LDS, ws);
}
extern "C" __global__ void __launch_bounds__(512) gemv_nvfp4_gum_bf16(const unsigned char* __restrict__ wg, const unsigned char* __restrict__ wu,
                                                                       const unsigned short* __restrict__ x, const float* __restrict__ gs_g,
                                                                       const float* __restrict__ gs_u, float* __restrict__ y,
                                                                       const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                       const int* __restrict__ m_p, int geo, const Workspace ws) {
    ENTER(wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p, m_p, geo);
    const int pairs = geo & 0xFFFFF;
    GemvArgs a = gemv_args(wg, wu, gs_g, gs_u, x, (size_t)pairs * CROW_PAIR_COLS, y, 0, pairs, k_dim_p, rows_p);
    gemv_m_dispatch<2, true, EPI_SILU_GU, CROW_MULTI_STRIPS_BF16>(a, rows_of(a, geo, m_p), 0, LDS, ws);
}

// ------------------------------------------------------------------ batched over token rows
// reference: gemv_fp4_b / gemv_fp4_b1k, engine/src/kernels.rs:154-189,1302-1337 and gemv_fp4_bs,
// :1022-1058.  grid.z = ceil(T / 4): each block decodes its weights once for up to 4 token rows.
// (gemv_fp4_b1k is the reference's 1024-thread variant of gemv_fp4_b for tensors of few rows; here the block shape follows
// K alone, so both names run the same body.)
__device__ __forceinline__ void gemv_tokens(const unsigned char* w, const float* x, const float* gs, float* y, int geo, const int* k_dim_p,
                                            const int* rows_p, const int* t_p, size_t y_stride, const Workspace& ws) {
    const int pairs = geo & 0xFFFFF, hint = (geo >> 20) & 0xF;
    const int t0 = (int)blockIdx.z * 4;
    const size_t k = (size_t)pairs * CROW_PAIR_COLS;
    GemvArgs a = gemv_args(w, nullptr, gs, nullptr, x + (size_t)t0 * k, k, y, y_stride, pairs, k_dim_p, rows_p);
    a.y_row0 = t0;
    int m;
    if (hint != 0) {  // the launcher knew the token count: every token group but the last is full, and the last holds `hint` rows
        m = blockIdx.z + 1 < gridDim.z ? 4 : hint;
        a.count_p = t_p;
        a.count_expect = 4 * ((int)gridDim.z - 1) + hint;
    } else {
        const int t_total = *t_p;
        if (t0 >= t_total) return;
        m = t_total - t0 < 4 ? t_total - t0 : 4;
    }
    gemv_m_dispatch<1, false, EPI_SCALE>(a, m, blockIdx.z, LDS, ws);
}
extern "C" __global__ void __launch_bounds__(512) gemv_fp4_b(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                              const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                              const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                              const int* __restrict__ t_p, int geo, const Workspace ws) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, t_p, geo);
    gemv_tokens(w, x, gs_ptr, y, geo, k_dim_p, rows_p, t_p, 0, ws);
}
extern "C" __global__ void __launch_bounds__(512) gemv_fp4_b1k(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                                const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                const int* __restrict__ t_p, int geo, const Workspace ws) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, t_p, geo);
    gemv_tokens(w, x, gs_ptr, y, geo, k_dim_p, rows_p, t_p, 0, ws);
}
extern "C" __global__ void __launch_bounds__(512) gemv_fp4_bs(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                               const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                               const int* __restrict__ k_dim_p, const int* __restrict__ y_stride_p,
                                                               const int* __restrict__ rows_p, const int* __restrict__ t_p, int geo, const Workspace ws) {
    ENTER(w, x, gs_ptr, y, k_dim_p, y_stride_p, rows_p, t_p, geo);
    const int y_stride = *y_stride_p;
    if (y_stride < *rows_p) {  // rows of y would overlap: refuse (uniform over the launch)
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
        return;
    }
    gemv_tokens(w, x, gs_ptr, y, geo, k_dim_p, rows_p, t_p, (size_t)y_stride, ws);
}

// ------------------------------------------------------------------ routed experts
// A slab pointer of zero is what a routing launch that refused its geometry leaves behind (the pointer tables start as
// zeros): every routed kernel reports it through the status word, uniformly per block and before any barrier, instead of
// reading weights through it.
#define CROW_REFUSE_NULL_SLAB(w)                                   \
    if ((w) == nullptr) {                                          \
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_GEO); \
        return;                                                    \
    }
// reference: gemv_fp4_ptrb, engine/src/kernels.rs:195-233.  grid.z = combo; ptrs[combo] is the
// device address of that combo's expert matrix in the tiled layout; x row = combo / x_div.
extern "C" __global__ void __launch_bounds__(1024) gemv_fp4_ptrb(const unsigned long long* __restrict__ ptrs, const float* __restrict__ x,
                                                                 const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                 const int* __restrict__ k_dim_p, const int* __restrict__ x_div_p,
                                                                 const int* __restrict__ x_stride_p, const int* __restrict__ rows_p, int geo, const Workspace ws) {
    ENTER(ptrs, x, gs_ptr, y, k_dim_p, x_div_p, x_stride_p, rows_p, geo);
    const int pairs = geo & 0xFFFFF;
    const int combo = (int)blockIdx.z;
    const unsigned char* w = (const unsigned char*)ptrs[combo];
    CROW_REFUSE_NULL_SLAB(w);
    GemvArgs a = gemv_args(w, nullptr, gs_ptr, nullptr, x + (size_t)(combo / *x_div_p) * *x_stride_p, 0, y, 0, pairs, k_dim_p, rows_p);
    a.y_row0 = combo;
    gemv_body<1, 1, false, EPI_SCALE>(a, blockIdx.z, LDS, ws);
}
// Fused routed gate|up + SwiGLU: the expert's fused tensor [2 I][H] holds gate in rows 0..I and up
// in rows I..2I (converter/tests/fixtures/cnq45m-index.tsv:351); h[combo][I] = silu(gate x) * up x.
// Replaces gemv_fp4_ptrb(gate_up) + silu_mul_combo of engine/src/gen.rs:4505-4517.  I % 16 == 0.
// byte offset of the `up` half inside a fused [2 I][K] slab
__device__ __forceinline__ size_t up_offset(int inter, int pairs) {
    return (size_t)(inter / CROW_STRIP_ROWS) * ((pairs + CROW_GROUP_PAIRS - 1) / CROW_GROUP_PAIRS) * CROW_GROUP_BYTES;
}
extern "C" __global__ void __launch_bounds__(1024) moe_gate_up_silu(const unsigned long long* __restrict__ ptrs, const float* __restrict__ x,
                                                                    const float* __restrict__ gs_ptr, float* __restrict__ h,
                                                                    const int* __restrict__ k_dim_p, const int* __restrict__ x_div_p,
                                                                    const int* __restrict__ x_stride_p, const int* __restrict__ inter_p, int geo, const Workspace ws) {
    ENTER(ptrs, x, gs_ptr, h, k_dim_p, x_div_p, x_stride_p, inter_p, geo);
    const int pairs = geo & 0xFFFFF;
    const int combo = (int)blockIdx.z, inter = *inter_p;  // (arrives with ptrs[combo]: no round trip of its own)
    const unsigned char* w = (const unsigned char*)ptrs[combo];
    CROW_REFUSE_NULL_SLAB(w);
    if (inter % CROW_STRIP_ROWS != 0) {  // gate and up are whole strips of the fused tensor
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
        return;
    }
    GemvArgs a = gemv_args(w, w + up_offset(inter, pairs), gs_ptr, gs_ptr, x + (size_t)(combo / *x_div_p) * *x_stride_p, 0, h, 0, pairs, k_dim_p, inter_p);
    a.y_row0 = combo;
    gemv_body<2, 1, false, EPI_SILU_GU>(a, blockIdx.z, LDS, ws);
}

// Fused routed down projection + weighted combine: y[t][row] += sum_j rw[t][j] * (gs * <down_{e(t,j)} row, h[t K + j]>),
// j ascending, each product and each add rounded on its own - the arithmetic of gemv_fp4_ptrb(down)
// followed by acc_combo (engine/src/gen.rs:4527-4531, engine/src/kernels.rs:1583-1592) in one launch.
// grid (ceil(H / 16), 1, T), block 64 * topk: wave j of a block takes combo t K + j and ALL columns of its strip.
extern "C" __global__ void __launch_bounds__(1024) moe_down_combine(const unsigned long long* __restrict__ ptrs, const float* __restrict__ h,
                                                                    const float* __restrict__ gs_ptr, const float* __restrict__ rw,
                                                                    float* __restrict__ y, const int* __restrict__ k_dim_p,
                                                                    const int* __restrict__ rows_p, int geo, const Workspace ws, const Geo model) {
    ENTER(ptrs, h, gs_ptr, rw, y, k_dim_p, rows_p, geo);
    const int pairs = geo & 0xFFFFF;
    constexpr int AREA = crow_gemv_lds_per_wave(1, false);
    const int topk = block_threads() >> 6;
    if (topk != model.topk || topk > 16) {
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_GEO);
        return;
    }
    const int k = pairs * CROW_PAIR_COLS, groups = (pairs + CROW_GROUP_PAIRS - 1) / CROW_GROUP_PAIRS;
    const int t = (int)blockIdx.z, strip = (int)blockIdx.x, j = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = lane_id();
    const int combo = t * topk + j;
    // dynamic LDS: zeros, then one f32 one-row staging area per wave; a wave's weighted result for wave 0 goes where its staged
    // activations were
    lds_p zero = LDS, areas = LDS + CROW_GEMV_ZERO_BYTES;
    const unsigned char* w = (const unsigned char*)ptrs[combo];
    // everything the epilogue needs is requested in the same round trip as the slab pointer: at one wave per SIMD nothing
    // hides a dependent load between the last product and the store (the row count, the caller's K, the routing weight, the
    // scale, and the old value of y that the result is added to)
    const int rows = *rows_p, k_word = *k_dim_p;
    const float gs = gs_ptr[0], weight = rw[combo];
    const int row = strip * CROW_STRIP_ROWS + lane;
    const bool writer = j == 0 && lane < 16 && row < rows;
    float y_old = 0.0f;
    if (writer) y_old = y[(size_t)t * rows + row];
    const size_t xoff[1] = {0};
    StripWalk<1, false> walk;
    // a routing launch that refused its geometry left zeros behind: no weights to read; the wave still joins the barriers below
    const int count = w != nullptr ? groups : 0;
    walk.init(w + (size_t)strip * groups * CROW_GROUP_BYTES, 0, k, h + (size_t)combo * k, xoff, areas + j * AREA, zero);
    walk.go(count, [&]() {
        for (int o = 16 * (int)threadIdx.x; o < CROW_GEMV_ZERO_BYTES; o += 16 * (topk << 6)) lds_store16(zero + o, 0, 0, 0, 0);
        __syncthreads();
    });
    float acc[1];
    walk.finish(acc);
    if (w == nullptr && lane == 0) atomicOr(ws.status, STATUS_BAD_GEO);
    if (lane < 16) ((lds_f)(areas + j * AREA))[lane] = weight * (acc[0] * gs);
    __syncthreads();
    if (!writer) return;
    if (k_word != k) {
        if (lane == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
        return;
    }
    float sum = 0.0f;
    for (int q = 0; q < topk; q++) sum = __fadd_rn(sum, ((lds_f)(areas + q * AREA))[lane]);
    y[(size_t)t * rows + row] = y_old + sum;
}

// ------------------------------------------------------------------ routed experts, grouped by expert (batches of many tokens)
// The per-combo kernels above read a routed expert's slab once per token that picked it.  For batches in which experts
// repeat, moe_group (misc_kernels.h) sorts the combos by expert and cuts them into tiles of at most four combos of one
// expert (the idea of moe_count / moe_plan / moe_scatter, engine/src/kernels.rs:3322-3384, in one launch); the two kernels
// below multiply a tile's slab once by its (up to) four rows, gathered through `perm`.  grid (strips, S, max tiles):
// blocks of tiles >= *n_tiles_p leave at once.  tiles[z] = (expert, first position in perm, combos, 0); table[2 e] /
// table[2 e + 1] = gate|up / down slab of expert e (the router's table).  Row m of a tile is combo c = perm[first + m]:
// it reads activation row c / *x_div_p and writes output row c.
extern "C" __global__ void __launch_bounds__(512) moe_gate_up_silu_grouped(const int4* __restrict__ tiles, const int* __restrict__ n_tiles_p,
                                                                             const int* __restrict__ perm, const unsigned long long* __restrict__ table,
                                                                             const float* __restrict__ x, const float* __restrict__ gs_ptr,
                                                                             float* __restrict__ h, const int* __restrict__ k_dim_p,
                                                                             const int* __restrict__ x_div_p, const int* __restrict__ x_stride_p,
                                                                             const int* __restrict__ inter_p, int geo, const Workspace ws) {
    ENTER(tiles, n_tiles_p, perm, table, x, gs_ptr, h, k_dim_p, x_div_p, x_stride_p, inter_p, geo);
    const int pairs = geo & 0xFFFFF;
    const int z = (int)blockIdx.z;
    if (z >= *n_tiles_p) return;
    const int4 tl = tiles[z];
    const int inter = *inter_p;
    const unsigned char* w = (const unsigned char*)table[2 * tl.x];
    CROW_REFUSE_NULL_SLAB(w);
    if (inter % CROW_STRIP_ROWS != 0) {
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
        return;
    }
    GemvArgs a = gemv_args(w, w + up_offset(inter, pairs), gs_ptr, gs_ptr, x, (size_t)*x_stride_p, h, 0, pairs, k_dim_p, inter_p);
    a.row_map = perm + tl.y, a.x_div = *x_div_p;
    gemv_m_dispatch<2, false, EPI_SILU_GU>(a, tl.z, blockIdx.z, LDS, ws);
}
// down slabs: x = h [combos][k_dim], y = eo [combos][rows]; acc_combo then adds the weighted rows per token
extern "C" __global__ void __launch_bounds__(512) moe_down_grouped(const int4* __restrict__ tiles, const int* __restrict__ n_tiles_p,
                                                                    const int* __restrict__ perm, const unsigned long long* __restrict__ table,
                                                                    const float* __restrict__ h, const float* __restrict__ gs_ptr,
                                                                    float* __restrict__ eo, const int* __restrict__ k_dim_p,
                                                                    const int* __restrict__ rows_p, int geo, const Workspace ws) {
    ENTER(tiles, n_tiles_p, perm, table, h, gs_ptr, eo, k_dim_p, rows_p, geo);
    const int pairs = geo & 0xFFFFF;
    const int z = (int)blockIdx.z;
    if (z >= *n_tiles_p) return;
    const int4 tl = tiles[z];
    const unsigned char* w = (const unsigned char*)table[2 * tl.x + 1];
    CROW_REFUSE_NULL_SLAB(w);
    GemvArgs a = gemv_args(w, nullptr, gs_ptr, nullptr, h, (size_t)pairs * CROW_PAIR_COLS, eo, 0, pairs, k_dim_p, rows_p);
    a.row_map = perm + tl.y, a.x_div = 1;
    gemv_m_dispatch<1, false, EPI_SCALE>(a, tl.z, blockIdx.z, LDS, ws);
}
// The two kernels above for strips of two to eight groups that one wave walks alone (K in 257 .. 2048 for gate|up, .. 1792 for
// down: this model's slabs), which the launcher starts in their place whenever the launch dimensions say so (one table entry,
// one name each): a block stages the tile's activation rows once and every wave streams runs of strips (gemv.h: TileWalk);
// crow_hip_launch_dims sizes the grid for it.  Here bits 24..31 of the geometry word = strips per wave.  Same bits.
#define CROW_TILE_DISPATCH(NR, EPI)                                      \
    switch (tl.z) {                                                      \
        case 1: tile_body<1, NR, EPI>(a, (geo >> 24) & 0xFF, LDS, ws); break; \
        case 2: tile_body<2, NR, EPI>(a, (geo >> 24) & 0xFF, LDS, ws); break; \
        case 3: tile_body<3, NR, EPI>(a, (geo >> 24) & 0xFF, LDS, ws); break; \
        case 4: tile_body<4, NR, EPI>(a, (geo >> 24) & 0xFF, LDS, ws); break; \
        default:                                                         \
            if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE); \
    }
extern "C" __global__ void __launch_bounds__(512) moe_gate_up_silu_grouped_tile(const int4* __restrict__ tiles, const int* __restrict__ n_tiles_p,
                                                                                  const int* __restrict__ perm, const unsigned long long* __restrict__ table,
                                                                                  const float* __restrict__ x, const float* __restrict__ gs_ptr,
                                                                                  float* __restrict__ h, const int* __restrict__ k_dim_p,
                                                                                  const int* __restrict__ x_div_p, const int* __restrict__ x_stride_p,
                                                                                  const int* __restrict__ inter_p, int geo, const Workspace ws) {
    ENTER(tiles, n_tiles_p, perm, table, x, gs_ptr, h, k_dim_p, x_div_p, x_stride_p, inter_p, geo);
    const int pairs = geo & 0xFFFFF;
    const int z = (int)blockIdx.z;
    if (z >= *n_tiles_p) return;
    const int4 tl = tiles[z];
    const int inter = *inter_p;
    const unsigned char* w = (const unsigned char*)table[2 * tl.x];
    CROW_REFUSE_NULL_SLAB(w);
    if (inter % CROW_STRIP_ROWS != 0) {
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
        return;
    }
    GemvArgs a = gemv_args(w, w + up_offset(inter, pairs), gs_ptr, gs_ptr, x, (size_t)*x_stride_p, h, 0, pairs, k_dim_p, inter_p);
    a.row_map = perm + tl.y, a.x_div = *x_div_p;
    CROW_TILE_DISPATCH(2, EPI_SILU_GU)
}
extern "C" __global__ void __launch_bounds__(512) moe_down_grouped_tile(const int4* __restrict__ tiles, const int* __restrict__ n_tiles_p,
                                                                         const int* __restrict__ perm, const unsigned long long* __restrict__ table,
                                                                         const float* __restrict__ h, const float* __restrict__ gs_ptr,
                                                                         float* __restrict__ eo, const int* __restrict__ k_dim_p,
                                                                         const int* __restrict__ rows_p, int geo, const Workspace ws) {
    ENTER(tiles, n_tiles_p, perm, table, h, gs_ptr, eo, k_dim_p, rows_p, geo);
    const int pairs = geo & 0xFFFFF;
    const int z = (int)blockIdx.z;
    if (z >= *n_tiles_p) return;
    const int4 tl = tiles[z];
    const unsigned char* w = (const unsigned char*)table[2 * tl.x + 1];
    CROW_REFUSE_NULL_SLAB(w);
    GemvArgs a = gemv_args(w, nullptr, gs_ptr, nullptr, h, (size_t)pairs * CROW_PAIR_COLS, eo, 0, pairs, k_dim_p, rows_p);
    a.row_map = perm + tl.y, a.x_div = 1;
    CROW_TILE_DISPATCH(1, EPI_SCALE)
}
#undef CROW_TILE_DISPATCH

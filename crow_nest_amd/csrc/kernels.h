// Kernel entry points of the library.  Names and argument lists follow the reference's kernel
// table (engine/src/kernels.rs:5135-5201, kernels_p2.rs) so that the call sites in
// engine/src/gen.rs keep their `launch_v(k.f(name), ..., &[args])` form; every argument is a
// device address, scalars are 4-byte device words (the reference's own convention,
// engine/src/cuda.rs:1-4).  Where an entry needs one more scalar than its reference twin
// (the row count, which the reference encodes in its grid) it is appended at the END of the
// list and named *_p like the others.
#pragma once
#include "gemv.h"

using namespace crow;

// The block's dynamic LDS (zeros, activation staging, wave hand-over: gemv.h); the launcher sizes it.
extern __shared__ uint4 crow_dyn_lds[];
#define LDS ((lds_p)crow_dyn_lds)
// First statement of every GEMV entry point: the workspace descriptor is fetched with the kernel arguments, in the
// first scalar round trip.  Left alone the compiler issues it after the shape words behind k_dim_p / rows_p have
// arrived, as a third dependent round trip in front of every wave's first weight load.
#define ENTER(...)                \
    const Workspace ws = g_ws;    \
    __builtin_amdgcn_sched_barrier(0)

// ------------------------------------------------------------------ dense GEMV (decode, one row)
// reference: gemv_nvfp4_w, engine/src/kernels_p2.rs:355-368
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_w(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                                const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                const int* __restrict__ k_dim_p, const int* __restrict__ rows_p) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p);
    GemvArgs a{{w, nullptr}, {gs_ptr, nullptr}, x, 0, y, 0, *k_dim_p, *rows_p, 1, nullptr};
    gemv_body<1, 1, false, EPI_SCALE, XRows<1, false>::value>(a, 0, LDS, ws);
}
// the same product on bf16 activations (exact widening), for models that keep their activations in bf16
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_w_bf16(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                                                     const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                     const int* __restrict__ k_dim_p, const int* __restrict__ rows_p) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p);
    GemvArgs a{{w, nullptr}, {gs_ptr, nullptr}, x, 0, y, 0, *k_dim_p, *rows_p, 1, nullptr};
    gemv_body<1, 1, true, EPI_SCALE, XRows<1, true>::value>(a, 0, LDS, ws);
}
// reference: gemv_fp4, engine/src/kernels.rs:118-151 (+ rows_p: the reference's grid.x is the row count)
extern "C" __global__ void __launch_bounds__(1024) gemv_fp4(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                            const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                            const int* __restrict__ k_dim_p, const int* __restrict__ rows_p) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p);
    GemvArgs a{{w, nullptr}, {gs_ptr, nullptr}, x, 0, y, 0, *k_dim_p, *rows_p, 1, nullptr};
    gemv_body<1, 1, false, EPI_SCALE, XRows<1, false>::value>(a, 0, LDS, ws);
}

// lm_head with the first stage of the greedy argmax fused in: logits[rows], and one candidate per 64-row
// tile kept in the library workspace; argmax_tiles(out_idx, rows_p) then picks the token from those
// ceil(rows / 64) candidates instead of re-reading all logits.  Together they replace lm_head_row +
// argmax_k (engine/src/gen.rs:4766-4784, engine/src/kernels.rs:4238-4260), same tie rule.
// out_idx is only a flag here (non-null selects the fused epilogue); argmax_tiles writes it.
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_w_argmax(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                                       const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                       const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                       int* __restrict__ out_idx) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, out_idx);
    GemvArgs a{{w, nullptr}, {gs_ptr, nullptr}, x, 0, y, 0, *k_dim_p, *rows_p, 1, out_idx};
    gemv_body<1, 1, false, EPI_SCALE, XRows<1, false>::value>(a, 0, LDS, ws);
}

// ------------------------------------------------------------------ fused gate/up + SiLU (decode)
// reference: gemv_nvfp4_gu, engine/src/kernels_p2.rs:372-389
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_gu(const unsigned char* __restrict__ wg, const unsigned char* __restrict__ wu,
                                                                 const float* __restrict__ x, const float* __restrict__ gs_g,
                                                                 const float* __restrict__ gs_u, float* __restrict__ y,
                                                                 const int* __restrict__ k_dim_p, const int* __restrict__ rows_p) {
    ENTER(wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p);
    GemvArgs a{{wg, wu}, {gs_g, gs_u}, x, 0, y, 0, *k_dim_p, *rows_p, 1, nullptr};
    gemv_body<2, 1, false, EPI_SILU_GU, XRows<1, false>::value, true>(a, 0, LDS, ws);
}

// the same on bf16 activations (exact widening)
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_gu_bf16(const unsigned char* __restrict__ wg, const unsigned char* __restrict__ wu,
                                                                      const unsigned short* __restrict__ x, const float* __restrict__ gs_g,
                                                                      const float* __restrict__ gs_u, float* __restrict__ y,
                                                                      const int* __restrict__ k_dim_p, const int* __restrict__ rows_p) {
    ENTER(wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p);
    GemvArgs a{{wg, wu}, {gs_g, gs_u}, x, 0, y, 0, *k_dim_p, *rows_p, 1, nullptr};
    gemv_body<2, 1, true, EPI_SILU_GU, XRows<1, true>::value, true>(a, 0, LDS, ws);
}

// ------------------------------------------------------------------ M <= 4 rows (MTP verify)
template <int NR, bool XBF16, int EPI>
__device__ __forceinline__ void gemv_m_dispatch(GemvArgs& a, unsigned z, lds_p lds, const Workspace& ws) {
    if (a.m < 1 || a.m > 4) {  // the reference's NVFP4_MMAX (engine/src/kernels_p2.rs:397-400); uniform over the launch
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
        return;
    }
    // one body per M keeps each row's operation sequence identical to the one-row kernel
    switch (a.m) {
        case 1: gemv_body<NR, 1, XBF16, EPI, XRows<4, XBF16>::value>(a, z, lds, ws); break;
        case 2: gemv_body<NR, 2, XBF16, EPI, XRows<4, XBF16>::value>(a, z, lds, ws); break;
        case 3: gemv_body<NR, 3, XBF16, EPI, XRows<4, XBF16>::value>(a, z, lds, ws); break;
        default: gemv_body<NR, 4, XBF16, EPI, XRows<4, XBF16>::value>(a, z, lds, ws); break;
    }
}
// reference: gemv_nvfp4_wm, engine/src/kernels_p2.rs:472-497
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_wm(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                                 const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                 const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                 const int* __restrict__ m_p) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, m_p);
    const int k = *k_dim_p, rows = *rows_p;
    GemvArgs a{{w, nullptr}, {gs_ptr, nullptr}, x, (size_t)k, y, (size_t)rows, k, rows, *m_p, nullptr};
    gemv_m_dispatch<1, false, EPI_SCALE>(a, 0, LDS, ws);
}
// reference: gemv_nvfp4_gum, engine/src/kernels_p2.rs:499-530
// (blocks of at most 8 waves: two weight tiles, four sets of split activation rows and their sums need more than 128 registers)
extern "C" __global__ void __launch_bounds__(512) gemv_nvfp4_gum(const unsigned char* __restrict__ wg, const unsigned char* __restrict__ wu,
                                                                  const float* __restrict__ x, const float* __restrict__ gs_g,
                                                                  const float* __restrict__ gs_u, float* __restrict__ y,
                                                                  const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                  const int* __restrict__ m_p) {
    ENTER(wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p, m_p);
    const int k = *k_dim_p, rows = *rows_p;
    GemvArgs a{{wg, wu}, {gs_g, gs_u}, x, (size_t)k, y, (size_t)rows, k, rows, *m_p, nullptr};
    gemv_m_dispatch<2, false, EPI_SILU_GU>(a, 0, LDS, ws);
}
// bf16-activation twins of the two verify kernels (X [M][k_dim] bf16, outputs f32)
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_wm_bf16(const unsigned char* __restrict__ w, const unsigned short* __restrict__ x,
                                                                      const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                      const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                      const int* __restrict__ m_p) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, m_p);
    const int k = *k_dim_p, rows = *rows_p;
    GemvArgs a{{w, nullptr}, {gs_ptr, nullptr}, x, (size_t)k, y, (size_t)rows, k, rows, *m_p, nullptr};
    gemv_m_dispatch<1, true, EPI_SCALE>(a, 0, LDS, ws);
}
extern "C" __global__ void __launch_bounds__(1024) gemv_nvfp4_gum_bf16(const unsigned char* __restrict__ wg, const unsigned char* __restrict__ wu,
                                                                       const unsigned short* __restrict__ x, const float* __restrict__ gs_g,
                                                                       const float* __restrict__ gs_u, float* __restrict__ y,
                                                                       const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                       const int* __restrict__ m_p) {
    ENTER(wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p, m_p);
    const int k = *k_dim_p, rows = *rows_p;
    GemvArgs a{{wg, wu}, {gs_g, gs_u}, x, (size_t)k, y, (size_t)rows, k, rows, *m_p, nullptr};
    gemv_m_dispatch<2, true, EPI_SILU_GU>(a, 0, LDS, ws);
}

// ------------------------------------------------------------------ batched over token rows
// reference: gemv_fp4_b / gemv_fp4_b1k, engine/src/kernels.rs:154-189,1302-1337 and gemv_fp4_bs,
// :1022-1058.  grid.z = ceil(T / 4): each block decodes its weights once for up to 4 token rows.
__device__ __forceinline__ void gemv_tokens(const unsigned char* w, const float* x, const float* gs, float* y, int k, int rows,
                                            int t_total, size_t y_stride, const Workspace& ws) {
    const int t0 = (int)blockIdx.z * 4;
    if (t0 >= t_total) return;
    GemvArgs a{{w, nullptr}, {gs, nullptr}, x + (size_t)t0 * k, (size_t)k, y + (size_t)t0 * y_stride, y_stride, k, rows,
               t_total - t0 < 4 ? t_total - t0 : 4, nullptr};
    gemv_m_dispatch<1, false, EPI_SCALE>(a, blockIdx.z, LDS, ws);
}
extern "C" __global__ void __launch_bounds__(1024) gemv_fp4_b(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                              const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                              const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                              const int* __restrict__ t_p) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, t_p);
    gemv_tokens(w, x, gs_ptr, y, *k_dim_p, *rows_p, *t_p, (size_t)*rows_p, ws);
}
extern "C" __global__ void __launch_bounds__(1024) gemv_fp4_b1k(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                                const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                const int* __restrict__ k_dim_p, const int* __restrict__ rows_p,
                                                                const int* __restrict__ t_p) {
    ENTER(w, x, gs_ptr, y, k_dim_p, rows_p, t_p);
    gemv_tokens(w, x, gs_ptr, y, *k_dim_p, *rows_p, *t_p, (size_t)*rows_p, ws);
}
extern "C" __global__ void __launch_bounds__(1024) gemv_fp4_bs(const unsigned char* __restrict__ w, const float* __restrict__ x,
                                                               const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                               const int* __restrict__ k_dim_p, const int* __restrict__ y_stride_p,
                                                               const int* __restrict__ rows_p, const int* __restrict__ t_p) {
    ENTER(w, x, gs_ptr, y, k_dim_p, y_stride_p, rows_p, t_p);
    gemv_tokens(w, x, gs_ptr, y, *k_dim_p, *rows_p, *t_p, (size_t)*y_stride_p, ws);
}

// ------------------------------------------------------------------ routed experts
// reference: gemv_fp4_ptrb, engine/src/kernels.rs:195-233.  grid.z = combo; ptrs[combo] is the
// device address of that combo's expert matrix in the tiled layout; x row = combo / x_div.
extern "C" __global__ void __launch_bounds__(1024) gemv_fp4_ptrb(const unsigned long long* __restrict__ ptrs, const float* __restrict__ x,
                                                                 const float* __restrict__ gs_ptr, float* __restrict__ y,
                                                                 const int* __restrict__ k_dim_p, const int* __restrict__ x_div_p,
                                                                 const int* __restrict__ x_stride_p, const int* __restrict__ rows_p) {
    ENTER(ptrs, x, gs_ptr, y, k_dim_p, x_div_p, x_stride_p, rows_p);
    const int combo = (int)blockIdx.z, rows = *rows_p;
    const unsigned char* w = (const unsigned char*)ptrs[combo];
    if (w == nullptr) {  // a router launch that refused its geometry leaves the pointer table untouched (zeros): refuse too
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_GEO);
        return;
    }
    GemvArgs a{{w, nullptr}, {gs_ptr, nullptr}, x + (size_t)(combo / *x_div_p) * *x_stride_p, 0, y + (size_t)combo * rows, 0, *k_dim_p, rows, 1, nullptr};
    gemv_body<1, 1, false, EPI_SCALE, XRows<1, false>::value>(a, blockIdx.z, LDS, ws);
}
// Fused routed gate|up + SwiGLU: the expert's fused tensor [2 I][H] holds gate in rows 0..I and up
// in rows I..2I (converter/tests/fixtures/cnq45m-index.tsv:351); h[combo][I] = silu(gate x) * up x.
// Replaces gemv_fp4_ptrb(gate_up) + silu_mul_combo of engine/src/gen.rs:4505-4517.  I % 64 == 0.
extern "C" __global__ void __launch_bounds__(1024) moe_gate_up_silu(const unsigned long long* __restrict__ ptrs, const float* __restrict__ x,
                                                                    const float* __restrict__ gs_ptr, float* __restrict__ h,
                                                                    const int* __restrict__ k_dim_p, const int* __restrict__ x_div_p,
                                                                    const int* __restrict__ x_stride_p, const int* __restrict__ inter_p) {
    ENTER(ptrs, x, gs_ptr, h, k_dim_p, x_div_p, x_stride_p, inter_p);
    const int combo = (int)blockIdx.z, inter = *inter_p, k = *k_dim_p;
    const unsigned char* w = (const unsigned char*)ptrs[combo];
    if (w == nullptr) {  // see gemv_fp4_ptrb
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_GEO);
        return;
    }
    const size_t up_off = (size_t)(inter / CROW_TILE_ROWS) * ((k + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS) * CROW_TILE_BYTES;
    GemvArgs a{{w, w + up_off}, {gs_ptr, gs_ptr}, x + (size_t)(combo / *x_div_p) * *x_stride_p, 0, h + (size_t)combo * inter, 0, k, inter, 1, nullptr};
    gemv_body<2, 1, false, EPI_SILU_GU, XRows<1, false>::value, true>(a, blockIdx.z, LDS, ws);
}

// Fused routed down projection + weighted combine: y[t][row] += sum_j rw[t][j] * (gs * <down_{e(t,j)} row, h[t K + j]>),
// j ascending, each product and each add rounded on its own - the arithmetic of gemv_fp4_ptrb(down)
// followed by acc_combo (engine/src/gen.rs:4527-4531, engine/src/kernels.rs:1583-1592) in one launch.
// grid (1, ceil(H / 64), T), block 64 * topk: wave j of a block takes combo t K + j.
extern "C" __global__ void __launch_bounds__(1024) moe_down_combine(const unsigned long long* __restrict__ ptrs, const float* __restrict__ h,
                                                                    const float* __restrict__ gs_ptr, const float* __restrict__ rw,
                                                                    float* __restrict__ y, const int* __restrict__ k_dim_p,
                                                                    const int* __restrict__ rows_p) {
    const int k = *k_dim_p, rows = *rows_p, topk = block_threads() >> 6;
    if (topk != g_geo.topk || topk > 16) {
        if (threadIdx.x == 0) atomicOr(g_ws.status, STATUS_BAD_GEO);
        return;
    }
    const int t = (int)blockIdx.z, rt = (int)blockIdx.y, j = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = lane_id();
    const int combo = t * topk + j;
    // dynamic LDS: zeros, 4 staging rows per wave (f32 activations, one token: hi, mid, lo, zero); a wave's weighted result
    // for wave 0 goes where its staged activations were
    typedef __attribute__((address_space(3))) float* lds_f;
    lds_p zero = LDS, xw = LDS + CROW_GEMV_ZERO_BYTES + j * (4 * CROW_GEMV_XROW_BYTES);
    if (threadIdx.x < CROW_GEMV_ZERO_BYTES / 16) lds_store16(zero + 16 * threadIdx.x, 0, 0, 0, 0);
    __syncthreads();
    const unsigned char* const w[2] = {(const unsigned char*)ptrs[combo], nullptr};
    float acc[1][1] = {{0.0f}};
    const size_t xoff[1] = {0};
    if (w[0] != nullptr) {
        tile_accumulate<1, 1, false>(w, rt, (k + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS, 0, 1, k, h + (size_t)combo * k, xoff, 1, xw, zero, acc);
    } else if (lane == 0) {  // a routing launch that refused its geometry left zeros behind: no weights to read; the wave
        atomicOr(g_ws.status, STATUS_BAD_GEO);  // still joins the barrier below
    }
    ((lds_f)xw)[lane] = rw[combo] * (acc[0][0] * gs_ptr[0]);
    __syncthreads();
    const int row = rt * CROW_TILE_ROWS + lane;
    if (j != 0 || row >= rows) return;
    float sum = 0.0f;
    for (int q = 0; q < topk; q++) sum = __fadd_rn(sum, ((lds_f)(LDS + CROW_GEMV_ZERO_BYTES + q * (4 * CROW_GEMV_XROW_BYTES)))[lane]);
    y[(size_t)t * rows + row] += sum;
}

// ------------------------------------------------------------------ routed experts, grouped by expert (batches of many tokens)
// The per-combo kernels above read a routed expert's slab once per token that picked it.  For batches in which experts
// repeat, moe_group (misc_kernels.h) sorts the combos by expert and cuts them into tiles of at most four combos of one
// expert (the idea of moe_count / moe_plan / moe_scatter, engine/src/kernels.rs:3322-3384, in one launch); the two kernels
// below multiply a tile's slab once by its (up to) four rows, gathered through `perm`.  grid (S, row tiles, max tiles):
// blocks of tiles >= *n_tiles_p leave at once.  tiles[z] = (expert, first position in perm, combos, 0); table[2 e] /
// table[2 e + 1] = gate|up / down slab of expert e (the router's table).  Row m of a tile is combo c = perm[first + m]:
// it reads activation row c / *x_div_p and writes output row c.
extern "C" __global__ void __launch_bounds__(512) moe_gate_up_silu_grouped(const int4* __restrict__ tiles, const int* __restrict__ n_tiles_p,
                                                                            const int* __restrict__ perm, const unsigned long long* __restrict__ table,
                                                                            const float* __restrict__ x, const float* __restrict__ gs_ptr,
                                                                            float* __restrict__ h, const int* __restrict__ k_dim_p,
                                                                            const int* __restrict__ x_div_p, const int* __restrict__ x_stride_p,
                                                                            const int* __restrict__ inter_p) {
    ENTER(tiles, n_tiles_p, perm, table, x, gs_ptr, h, k_dim_p, x_div_p, x_stride_p, inter_p);
    const int z = (int)blockIdx.z;
    if (z >= *n_tiles_p) return;
    const int4 tl = tiles[z];
    const int inter = *inter_p, k = *k_dim_p;
    const unsigned char* w = (const unsigned char*)table[2 * tl.x];
    const size_t up_off = (size_t)(inter / CROW_TILE_ROWS) * ((k + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS) * CROW_TILE_BYTES;
    GemvArgs a{{w, w + up_off}, {gs_ptr, gs_ptr}, x, (size_t)*x_stride_p, h, (size_t)inter, k, inter, tl.z, nullptr, perm + tl.y, *x_div_p};
    gemv_m_dispatch<2, false, EPI_SILU_GU>(a, blockIdx.z, LDS, ws);
}
// down slabs: x = h [combos][k_dim], y = eo [combos][rows]; acc_combo then adds the weighted rows per token
extern "C" __global__ void __launch_bounds__(1024) moe_down_grouped(const int4* __restrict__ tiles, const int* __restrict__ n_tiles_p,
                                                                    const int* __restrict__ perm, const unsigned long long* __restrict__ table,
                                                                    const float* __restrict__ h, const float* __restrict__ gs_ptr,
                                                                    float* __restrict__ eo, const int* __restrict__ k_dim_p,
                                                                    const int* __restrict__ rows_p) {
    ENTER(tiles, n_tiles_p, perm, table, h, gs_ptr, eo, k_dim_p, rows_p);
    const int z = (int)blockIdx.z;
    if (z >= *n_tiles_p) return;
    const int4 tl = tiles[z];
    const int k = *k_dim_p, rows = *rows_p;
    GemvArgs a{{(const unsigned char*)table[2 * tl.x + 1], nullptr}, {gs_ptr, nullptr}, h, (size_t)k, eo, (size_t)rows, k, rows, tl.z, nullptr, perm + tl.y, 1};
    gemv_m_dispatch<1, false, EPI_SCALE>(a, blockIdx.z, LDS, ws);
}

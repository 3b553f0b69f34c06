/*
 * The kernel table of libcrow_hip.so: every name crow_hip_module_get / crow_hip_get_function resolves, the values
 * crow_hip_launch expects for it (in order, each a 64-bit device address; `*_p` = address of a 4-byte device word, as the
 * reference's Params words), and the reference kernel whose call sites it serves.
 *
 * This header declares no C symbols: the kernels are reached by name through crow_hip_launch, exactly as the reference
 * reaches its kernels through Kernels::f(name) + launch_v (engine/src/kernels.rs:5234,5296).  Include it with CROW_KERNEL
 * defined to walk the table:
 *     #define CROW_KERNEL(name, n_values) ...
 *     #include "crow_kernels.h"
 * Without a definition every line expands to nothing.  Grid and block sizes always come from crow_hip_launch_dims.
 *
 * Conventions shared by all entries:
 *   w, wg, wu   NVFP4 tensors in the library's tiled layout (crow_hip_repack_nvfp4), never raw container bytes
 *   gs, gs_*    one f32 per tensor: the global scale (PW::Fp4's second word, engine/src/gen.rs:234-237)
 *   x           activations, row-major [tokens][k_dim]: f32 unless the entry is a *_bf16 twin (then bf16); 16-byte aligned
 *   y           f32 outputs, row-major [tokens][rows]
 *   A shape a kernel cannot serve sets a bit of the device status word (read by crow_hip_status) and the launch
 *   writes nothing; no kernel traps.
 */
#ifndef CROW_KERNEL
#define CROW_KERNEL(name, n_values)
#define CROW_KERNEL_DEFAULTED_
#endif

/* ---- dense GEMV, one token ------------------------------------------------------------------------------------------ */
/* w, x, gs, y, k_dim_p, rows_p.  gemv_nvfp4_w of engine/src/kernels_p2.rs:304-368 (rows_p appended: the reference reads
 * the row count off its grid). */
CROW_KERNEL(gemv_nvfp4_w, 6)
CROW_KERNEL(gemv_nvfp4_w_bf16, 6) /* the same on bf16 x */
/* w, x, gs, y, k_dim_p, rows_p.  gemv_fp4 of engine/src/kernels.rs:118-152 (the older one-block-per-row entry point the
 * engine still calls for some tensors); same arithmetic as gemv_nvfp4_w here. */
CROW_KERNEL(gemv_fp4, 6)
/* w, x, gs, y(logits), k_dim_p, rows_p, out_idx.  lm_head_row (engine/src/gen.rs:4766-4784) and argmax_k
 * (engine/src/kernels.rs:4238-4260) in one call: logits[rows] and out_idx[0] = the greedy token, same tie order as
 * argmax_k.  Each block leaves its strip's candidate in the library's scratch memory; crow_hip_launch starts a one-block
 * finishing kernel right behind the GEMV (on the same stream, also under capture) that writes the token. */
CROW_KERNEL(gemv_nvfp4_w_argmax, 7)
CROW_KERNEL(argmax_k, 3)     /* logits, out_idx, n_p.  engine/src/kernels.rs:4238-4260 */

/* ---- fused gate / up + SiLU ----------------------------------------------------------------------------------------- */
/* wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p.  gemv_nvfp4_gu of kernels_p2.rs:372-389: y = silu(gate x) * (up x). */
CROW_KERNEL(gemv_nvfp4_gu, 8)
CROW_KERNEL(gemv_nvfp4_gu_bf16, 8)

/* ---- M <= 4 token rows (speculative verify) ----------------------------------------------------------------------- */
/* w, x, gs, y, k_dim_p, rows_p, m_p.  gemv_nvfp4_wm of kernels_p2.rs:397-497; *m_p in 1..4 (NVFP4_MMAX), else the status
 * word gets the bad-shape bit.  Row m of the result is bit-identical to a one-token launch on row m of x. */
CROW_KERNEL(gemv_nvfp4_wm, 7)
CROW_KERNEL(gemv_nvfp4_wm_bf16, 7)
/* wg, wu, x, gs_g, gs_u, y, k_dim_p, rows_p, m_p.  gemv_nvfp4_gum of kernels_p2.rs:499-530. */
CROW_KERNEL(gemv_nvfp4_gum, 9)
CROW_KERNEL(gemv_nvfp4_gum_bf16, 9)
/* w, x, gs, y, k_dim_p, rows_p, t_p.  gemv_fp4_b / gemv_fp4_b1k of kernels.rs:154-189,1302-1337: any token count t,
 * four tokens per grid.z slice (rows_p and t_p appended). */
CROW_KERNEL(gemv_fp4_b, 7)
CROW_KERNEL(gemv_fp4_b1k, 7)
/* w, x, gs, y, k_dim_p, y_stride_p, rows_p, t_p.  gemv_fp4_bs of kernels.rs:1022-1058: as gemv_fp4_b with a row stride
 * on y. */
CROW_KERNEL(gemv_fp4_bs, 8)

/* ---- routed experts ------------------------------------------------------------------------------------------------- */
/* logits, bitmap, ids, wts, gu_ptrs, dn_ptrs, table, cold_mask, counters, sel_counts.  router_top10 of
 * kernels.rs:3109-3184: softmax, top-k with ties to the lowest id, renormalised weights, per-combo slab addresses gathered
 * from table[E][2].  Geometry (experts, top-k) from crow_hip_set_geo. */
CROW_KERNEL(router_top10, 10)
/* ptrs, x, gs, y, k_dim_p, x_div_p, x_stride_p, rows_p.  gemv_fp4_ptrb of kernels.rs:195-233: combo c multiplies the slab
 * at ptrs[c] by row c / *x_div_p of x (rows_p appended). */
CROW_KERNEL(gemv_fp4_ptrb, 8)
CROW_KERNEL(silu_mul_combo, 3) /* h1, h2, n_p.  kernels.rs:1562-1581 */
CROW_KERNEL(acc_combo, 3)      /* x, rw, y.     kernels.rs:1583-1592 */
/* ptrs, x, gs, h, k_dim_p, x_div_p, x_stride_p, inter_p.  gemv_fp4_ptrb on a fused gate_up slab + silu_mul_combo in one
 * launch: h[c][i] = silu(gate_c x)[i] * (up_c x)[i]. */
CROW_KERNEL(moe_gate_up_silu, 8)
/* logits, table, x, gs, h, ids, wts, dn_ptrs, k_dim_p, x_stride_p, inter_p.  router_top10 + moe_gate_up_silu in one launch:
 * every block works out its token's routing itself and takes its slab from table[2 e]; one block per token writes ids, wts
 * and dn_ptrs (table[2 e + 1]) for moe_down_combine.  Same routing, same h as the two launches it replaces. */
CROW_KERNEL(moe_route_gate_up_silu, 11)
/* ptrs, h, gs, rw, y, k_dim_p, rows_p.  gemv_fp4_ptrb on the down slabs + acc_combo in one launch: y[t] = sum over the
 * token's combos j, in j order, of rw[t][j] * (down_j h_j). */
CROW_KERNEL(moe_down_combine, 7)

/* routed experts grouped by expert, for batches in which experts repeat (the idea of moe_count / moe_plan / moe_scatter,
 * kernels.rs:3322-3384, without the staging of cold experts):
 * moe_group: ids, n_p, perm, tiles, n_tiles, max_tiles_p.  One block sorts the n <= 4096 combos by expert (stable) and cuts
 *   them into tiles (expert, first position in perm, combos <= 4, 0); sets the bad-geometry bit for an id outside
 *   0 .. experts - 1 and the workspace bit when more than *max_tiles_p tiles would be needed (then *n_tiles = 0).
 * moe_gate_up_silu_grouped: tiles, n_tiles_p, perm, table, x, gs, h, k_dim_p, x_div_p, x_stride_p, inter_p.
 * moe_down_grouped: tiles, n_tiles_p, perm, table, h, gs, eo, k_dim_p, rows_p (acc_combo then combines eo per token).
 *   grid.z = an upper bound of the tile count (crow_hip_launch_dims with z = that bound); blocks beyond *n_tiles_p leave. */
CROW_KERNEL(moe_group, 6)
CROW_KERNEL(moe_gate_up_silu_grouped, 11)
CROW_KERNEL(moe_down_grouped, 9)

/* ---- batched GEMM on the matrix cores (bf16 x, f32 y) ------------------------------------------------------------- */
/* w, x, gs, y, k_dim_p, rows_p, m_p.  The dense NVFP4 GEMM of kernels_glm5_moe.cu:310-543 (gemm_fp4_dense's list minus
 * the quantised-activation buffer: x is bf16).  gemm_nvfp4_bf16_m16 serves *m_p <= 16 only; the others take any m
 * and differ in tiling (32, 48, 64, 96, 128 tokens per block); crow_hip_gemm_kernel names the one to use. */
CROW_KERNEL(gemm_nvfp4_bf16, 7)
/* the same product in blocks of eight waves (two per SIMD) x 48 / 64 / 80 / 96 tokens: what crow_hip_gemm_kernel picks from a few
 * hundred tokens on */
CROW_KERNEL(gemm_nvfp4_bf16_w48, 7)
CROW_KERNEL(gemm_nvfp4_bf16_w64, 7)
CROW_KERNEL(gemm_nvfp4_bf16_w80, 7)
CROW_KERNEL(gemm_nvfp4_bf16_w96, 7)
CROW_KERNEL(gemm_nvfp4_bf16_m96, 7)
CROW_KERNEL(gemm_nvfp4_bf16_m64, 7)
CROW_KERNEL(gemm_nvfp4_bf16_m48, 7)
CROW_KERNEL(gemm_nvfp4_bf16_m32, 7)
CROW_KERNEL(gemm_nvfp4_bf16_m16, 7)

/* ---- BF16 weights the container keeps unquantised (router, MTP head) ---------------------------------------------- */
/* w(bf16 [rows][k_dim]), x, y, k_dim_p, rows_p.  gemv_bf16_w of kernels.rs:1130-1157; tokens on grid.y. */
CROW_KERNEL(gemv_bf16_w, 5)
/* the block-per-row forms of the same product, gemv_bf16 (one token, kernels.rs:1061-1077: the bf16 lm_head of gen.rs:4780)
 * and gemv_bf16_b (grid.y tokens, kernels.rs:1080-1098: the GLM5 router of glm5_moe.rs:731), + rows_p: the reference's
 * grid.x is the row count.  Launched with the dims of gemv_bf16_w. */
CROW_KERNEL(gemv_bf16, 5)
CROW_KERNEL(gemv_bf16_b, 5)
/* w(f32 [rows][k_dim]), x, y, k_dim_p, rows_p.  gemv_b of kernels.rs:97-115 (the router projection of gen.rs:4182), + rows_p;
 * k_dim a multiple of 4; tokens on grid.y. */
CROW_KERNEL(gemv_b, 5)
/* w(bf16), x, y, k_dim_p, rows_p.  gemv_bf16_ws of kernels.rs:1430-1458: gemv_bf16_w with the sigmoid applied at the store. */
CROW_KERNEL(gemv_bf16_ws, 5)
/* w(bf16), x, y, k_dim_p, y_stride_p, rows_p.  gemv_bf16_bs of kernels.rs:1100-1124: gemv_bf16_b writing y[t * *y_stride_p + row]
 * (two tensors into one [t][stride] buffer), + rows_p. */
CROW_KERNEL(gemv_bf16_bs, 6)

/* ---- layout and decode ---------------------------------------------------------------------------------------------- */
CROW_KERNEL(repack_nvfp4, 4)        /* src(container bytes), dst(tiled), rows_p, k_dim_p: what crow_hip_repack_nvfp4 launches */
CROW_KERNEL(unpack_nvfp4, 4)        /* src(tiled), dst(container bytes), rows_p, k_dim_p */
CROW_KERNEL(dequant_nvfp4_tiled, 5) /* w, gs, out(f32 [rows][k_dim]), rows_p, k_dim_p: bit-exact decode (cnq.rs:1298-1308) */
CROW_KERNEL(dequant_fp4_flat, 4)    /* w(raw container bytes), gs, out, n_p.  dequant_fp4_flat of kernels.rs:1460, same list */

/* ---- measurement only (not part of the drop-in set: the engine never asks for these) --------------------------------- */
/* w(raw container bytes), x, gs, y, k_dim_p, rows_p.  The one-row GEMV written the reference's way (kernels_p2.rs:304-368: lanes
 * across the columns, f32 multiply-adds on decoded weights, no matrix instructions), 1 / 2 / 4 rows per 16-lane group: the A/B
 * behind the choice of the matrix cores for one activation row (bench.py reports it). */
CROW_KERNEL(gemv_nvfp4_w_valu1, 6)
CROW_KERNEL(gemv_nvfp4_w_valu2, 6)
CROW_KERNEL(gemv_nvfp4_w_valu4, 6)

#ifdef CROW_KERNEL_DEFAULTED_
#undef CROW_KERNEL
#undef CROW_KERNEL_DEFAULTED_
#endif

/*
 * CPU oracle for the NVFP4 weight x activation path.  TEST INFRASTRUCTURE ONLY.
 *
 * This library restates, in plain C, the arithmetic of the reference's own CPU NVFP4 path and
 * of the small kernels around it, so that the HIP path can be checked against it.  Nothing in
 * the product may link or call it: only tests, the smoke check and the bench's CPU-baseline
 * leg do.  Every function names the reference lines it follows (paths are into the reference
 * checkout).  The reference is Rust and there is no Rust toolchain here, so there is no
 * oracle/_ref build; the restatement is pinned by the reference's own fixtures instead (see
 * the header comment of nvfp4_oracle.c for which check pins which function).
 *
 * All sizes are in elements unless a name ends in _bytes.  Return value 0 = ok, <0 = shape
 * error (the reference returns Err(String) for the same conditions).
 */
#ifndef NVFP4_ORACLE_H
#define NVFP4_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define NVFP4_BLOCK_BYTES 36
#define NVFP4_BLOCK_VALUES 64

/* ---- format (engine/src/cnq.rs:1241-1308, engine/src/cpu_nvfp4.rs:88-105) ---- */
float orc_e2m1(uint32_t nibble);
float orc_ue4m3(uint32_t byte);
uint8_t orc_scale_rule(uint8_t byte);
void orc_scale_lut(float global_scale, float lut[256]);
/* container-exact decode, NO 0x7F rule (cnq.rs:1298-1308, converter/src/main.rs:198-212) */
void orc_dequant_raw(const uint8_t* blocks, size_t n_blocks, float gs, float* out);
/* the decode the CPU path computes with: 0x7F -> 0x7E first (cpu_nvfp4.rs:98-105) */
void orc_dequant(const uint8_t* blocks, size_t n_blocks, float gs, float* out);
size_t orc_byte_len(size_t rows, size_t cols);

/* ---- encoder, ceil mode (converter/src/main.rs:141-169,404-410,550-664) ---- */
uint32_t orc_encode_ue4m3_ceil(float v);
/* values: n floats, n % 64 == 0; out: n/64*36 bytes; returns the global scale */
float orc_quantize_ceil(const float* values, size_t n, uint8_t* out);

/* ---- the CPU path (cpu_nvfp4.rs:181-427) ---- */
/* path: 0 = scalar, 1 = AVX2 (bit-identical by construction); threads >= 1 */
int orc_gemv(const uint8_t* w, size_t rows, size_t cols, float gs, const float* x, size_t tokens,
             float* y, int threads, int path);
int orc_expert_ffn(const uint8_t* gate, float gs_g, const uint8_t* up, float gs_u, const uint8_t* down,
                   float gs_d, size_t hidden, size_t inter, const float* x, size_t tokens, float* y,
                   int threads, int path);
/* dense FFN with the clamped SwiGLU of engine/src/glm5_moe.rs:141-154,271-278 (limit <= 0: no clamp) */
int orc_ffn_clamped(const uint8_t* gate, float gs_g, const uint8_t* up, float gs_u, const uint8_t* down,
                    float gs_d, size_t hidden, size_t inter, float limit, const float* x, size_t tokens,
                    float* y, int threads, int path);
/* f64 dequantize-then-dot and sum|w x| (cpu_nvfp4.rs:491-514); rule != 0 applies 0x7F -> 0x7E */
void orc_gemv_f64(const uint8_t* w, size_t rows, size_t cols, float gs, const float* x, size_t tokens,
                  int rule, double* y, double* sum_abs);
double orc_gamma(size_t cols);

/* ---- epilogues and the small kernels around the GEMV ---- */
/* silu(g) * u = g / (1 + exp(-g)) * u in f32 (cpu_nvfp4.rs:404, kernels_p2.rs:386-387) */
float orc_silu_mul(float g, float u);
/* [C][2I] -> [C][I] (kernels.rs:1562-1570) */
void orc_silu_mul_combo(const float* h1, size_t combos, size_t inter, float* h2);
/* y[t][c] += sum_j rw[t][j] * x[t*topk+j][c], j ascending (kernels.rs:1583-1592) */
void orc_acc_combo(const float* x, const float* rw, size_t tokens, size_t topk, size_t hidden, float* y);
/* softmax + top-k, lowest index on ties, renormalised (kernels.rs:3109-3184) */
void orc_router_topk(const float* logits, size_t tokens, size_t experts, size_t topk, int32_t* ids, float* wts);
/* greedy argmax with the reference's tie rule (kernels.rs:4238-4260): 1024 strided scanners, then a
 * halving tree that takes the right slot only when strictly greater */
int32_t orc_argmax_ref(const float* logits, size_t n);
/* whole MoE layer of config 2 (engine/src/gen.rs:4168-4534 call order, shared expert left out):
 * gate_up [E][2I][H] (rows 0..I gate, I..2I up), down [E][H][I], one gs per tensor */
int orc_moe_layer(const uint8_t* gate_up, float gs_gu, const uint8_t* down, float gs_dn, size_t experts,
                  size_t hidden, size_t inter, const float* x, const float* logits, size_t tokens,
                  size_t topk, int32_t* ids, float* wts, float* y, int threads, int path);

/* bf16 helpers used by the tests for configs whose X is bf16 */
uint16_t orc_f32_to_bf16(float v);   /* RNE, kernels.rs:67-71 */
float orc_bf16_to_f32(uint16_t b);

#ifdef __cplusplus
}
#endif
#endif

// Load-time repack, dequant, and the small kernels around the GEMVs (router, SwiGLU, combine, argmax).
#pragma once
#include "device_common.h"

using namespace crow;

#define CROW_STATUS_BAD_SCALE_BYTE 8u

// ------------------------------------------------------------------ container <-> tiled
// One 64-thread block per group (blockIdx.x = group, blockIdx.y = strip); thread l moves the 36-byte container block
// (strip row l % 16, block l / 16 of the group's four).  Load-time work: neither the strided 36-byte reads nor the
// scattered 4-byte writes are coalesced, and they need not be.
extern "C" __global__ void __launch_bounds__(64) repack_nvfp4(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst,
                                                              const int* __restrict__ rows_p, const int* __restrict__ k_dim_p) {
    const int rows = *rows_p, k = *k_dim_p;
    const int groups = (k + CROW_GROUP_COLS - 1) / CROW_GROUP_COLS, bpr = k / CROW_BLOCK_VALUES;
    const int gi = (int)blockIdx.x, strip = (int)blockIdx.y, lane = lane_id();
    const int r = lane & 15, b = lane >> 4;
    const int row = strip * CROW_STRIP_ROWS + r, blk = gi * 4 + b;
    unsigned char* grp = dst + ((size_t)strip * groups + gi) * CROW_GROUP_BYTES;
    unsigned q[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
    if (row < rows && blk < bpr) {
        const unsigned* sq = (const unsigned*)(src + ((size_t)row * bpr + blk) * CROW_BLOCK_BYTES);
#pragma unroll
        for (int i = 0; i < 9; i++) q[i] = sq[i];
    }
    bool bad = false;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        unsigned v = (q[0] >> (8 * i)) & 0xFFu;
        if (v == 0xFFu) bad = true;
        v &= 0x7Fu;
        if (v == 0x7Fu) v = 0x7Eu;
        grp[crow_group_scale_offset((unsigned)r, (unsigned)(4 * b + i))] = (unsigned char)v;
    }
#pragma unroll
    for (int wd = 0; wd < 8; wd++) *(unsigned*)(grp + crow_group_code_offset((unsigned)r, (unsigned)(8 * b + wd))) = q[1 + wd];
    if (bad) atomicOr(g_ws.status, CROW_STATUS_BAD_SCALE_BYTE);
}

// The inverse: tiled -> container bytes (scale bytes come back canonical: 0x7F has become 0x7E and
// bit 7 is cleared; everything else is byte-identical to what was repacked).
extern "C" __global__ void __launch_bounds__(64) unpack_nvfp4(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst,
                                                              const int* __restrict__ rows_p, const int* __restrict__ k_dim_p) {
    const int rows = *rows_p, k = *k_dim_p;
    const int groups = (k + CROW_GROUP_COLS - 1) / CROW_GROUP_COLS, bpr = k / CROW_BLOCK_VALUES;
    const int gi = (int)blockIdx.x, strip = (int)blockIdx.y, lane = lane_id();
    const int r = lane & 15, b = lane >> 4;
    const int row = strip * CROW_STRIP_ROWS + r, blk = gi * 4 + b;
    if (row >= rows || blk >= bpr) return;
    const unsigned char* grp = src + ((size_t)strip * groups + gi) * CROW_GROUP_BYTES;
    unsigned* q = (unsigned*)(dst + ((size_t)row * bpr + blk) * CROW_BLOCK_BYTES);
    unsigned s4 = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) s4 |= (unsigned)grp[crow_group_scale_offset((unsigned)r, (unsigned)(4 * b + i))] << (8 * i);
    q[0] = s4;
#pragma unroll
    for (int wd = 0; wd < 8; wd++) q[1 + wd] = *(const unsigned*)(grp + crow_group_code_offset((unsigned)r, (unsigned)(8 * b + wd)));
}

// Dequantise a tiled tensor to f32 [rows][k_dim]: w = e2m1(code) * f32(ue4m3(scale) * gs), the two
// roundings of the reference decode in that order (engine/src/cnq.rs:1298-1308 with the scale rule of
// cpu_nvfp4.rs:98-105 already applied by the repacker).  Same grid as repack_nvfp4: thread l decodes the 64 values of
// strip row l % 16, container block l / 16 of the group.
extern "C" __global__ void __launch_bounds__(64) dequant_nvfp4_tiled(const unsigned char* __restrict__ w, const float* __restrict__ gs_ptr,
                                                                     float* __restrict__ out, const int* __restrict__ rows_p,
                                                                     const int* __restrict__ k_dim_p) {
    const int rows = *rows_p, k = *k_dim_p;
    const int groups = (k + CROW_GROUP_COLS - 1) / CROW_GROUP_COLS;
    const int gi = (int)blockIdx.x, strip = (int)blockIdx.y, lane = lane_id();
    const int r = lane & 15, b = lane >> 4;
    const int row = strip * CROW_STRIP_ROWS + r, col_b = gi * CROW_GROUP_COLS + b * CROW_BLOCK_VALUES;
    if (row >= rows || col_b >= k) return;
    const float gs = gs_ptr[0];
    const unsigned char* grp = w + ((size_t)strip * groups + gi) * CROW_GROUP_BYTES;
    for (int i = 0; i < 4; i++) {
        const int sb = 4 * b + i;
        const unsigned byte = grp[crow_group_scale_offset((unsigned)r, (unsigned)sb)];
        const float sf = __builtin_amdgcn_cvt_f32_fp8((int)byte, 0) * gs;
        float* o = out + (size_t)row * k + col_b + 16 * i;
        for (int d = 0; d < 2; d++) {
            const unsigned wd = *(const unsigned*)(grp + crow_group_code_offset((unsigned)r, (unsigned)(2 * sb + d)));
            for (int j = 0; j < 8; j++) {
                const unsigned nib = (wd >> (4 * j)) & 0xFu;
                const f32x2 v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(nib, 1.0f, 0);
                o[d * 8 + j] = v.x * sf;
            }
        }
    }
}

// reference: dequant_fp4_flat, engine/src/kernels.rs:1460-1471 - CONTAINER layout, raw decode
// (no scale rule: 0x7F reads 480, bit 7 ignored), one thread per value.
extern "C" __global__ void dequant_fp4_flat(const unsigned char* __restrict__ w, const float* __restrict__ gs_ptr,
                                            float* __restrict__ out, const int* __restrict__ n_p) {
    const int i = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (i >= *n_p) return;
    const int b = i >> 6, idx = i & 63;
    const unsigned char* blk = w + (size_t)b * CROW_BLOCK_BYTES;
    // (byte & 0x7F) << 20 is the f32 whose value is ue4m3(byte) * 2^-120, subnormal ladder included
    const float u = __uint_as_float(((unsigned)blk[idx >> 4] & 0x7Fu) << 20) * 0x1p120f;
    const float s = u * gs_ptr[0];
    const unsigned byte = blk[4 + (idx >> 1)];
    const unsigned nib = (idx & 1) ? (byte >> 4) : (byte & 0xFu);
    const f32x2 v = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(nib, 1.0f, 0);
    out[i] = v.x * s;
}

// ------------------------------------------------------------------ measurement only: what a pure read of the same bytes takes
// The textbook streaming read, for comparison with the pattern below: every lane 16 contiguous bytes per load (a wave 1 KB per
// instruction), eight loads in flight per lane, the grid striding over the buffer; NT = non-temporal loads or plain ones.
template <bool NT>
__device__ __forceinline__ void pure_read_flat_body(const uint4* __restrict__ w, size_t n16, unsigned* __restrict__ sink) {
    const size_t total = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    unsigned q = 0;
    for (; i + 7 * total < n16; i += 8 * total) {
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = NT ? stream_load_v(w + i + j * total) : *(const u32x4*)(w + i + j * total);
#pragma unroll
        for (int j = 0; j < 8; j++) q ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
    }
    for (; i < n16; i += total) {
        const u32x4 v = NT ? stream_load_v(w + i) : *(const u32x4*)(w + i);
        q ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (q == 0x9E3779B9u) *sink = q;  // keeps the loads alive; practically never taken
}
extern "C" __global__ void __launch_bounds__(1024) pure_read_flat_nt(const uint4* __restrict__ w, size_t n16, unsigned* __restrict__ sink) {
    pure_read_flat_body<true>(w, n16, sink);
}
extern "C" __global__ void __launch_bounds__(1024) pure_read_flat(const uint4* __restrict__ w, size_t n16, unsigned* __restrict__ sink) {
    pure_read_flat_body<false>(w, n16, sink);
}

// Reads `units` 2304-byte groups exactly as the GEMVs request them (one dword and two 16-byte non-temporal loads per lane and
// group, four groups in flight per wave) and does nothing else: the chip's ceiling for this access pattern, measured beside
// the kernels by the benchmark.  Group i goes to wave i % (all waves of the grid), so any grid covers any size.
extern "C" __global__ void __launch_bounds__(1024) pure_read_groups(const unsigned char* __restrict__ w, unsigned units, unsigned* __restrict__ sink) {
    const int lane = lane_id();
    const unsigned waves = gridDim.x * (blockDim.x >> 6), wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const unsigned count = units > wave ? (units - wave + waves - 1) / waves : 0u;
    const unsigned char* p = w + (size_t)wave * CROW_GROUP_BYTES;
    const size_t step = (size_t)waves * CROW_GROUP_BYTES;
    unsigned sc[4];
    u32x4 c0[4], c1[4];
    unsigned q = 0;
    auto issue = [&](int j) {
        sc[j] = stream_load_u32((const unsigned*)p + lane);
        c0[j] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES) + lane);
        c1[j] = stream_load_v((const uint4*)(p + CROW_GROUP_SCALE_BYTES + 1024) + lane);
        p += step;
    };
    auto use = [&](int j) { q ^= sc[j] ^ c0[j].x ^ c0[j].w ^ c1[j].y ^ c1[j].z; };
    if (count >= 4) {
#pragma unroll
        for (int j = 0; j < 4; j++) issue(j);
        unsigned left = count - 4;
        for (; left >= 4; left -= 4) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                use(j);
                issue(j);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            use(j);
            if ((unsigned)j < left) issue(j);
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
            if ((unsigned)j < left) use(j);
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++)
            if ((unsigned)j < count) issue(j);
#pragma unroll
        for (int j = 0; j < 4; j++)
            if ((unsigned)j < count) use(j);
    }
    if (q == 0x12345677u) sink[0] = q;  // (keeps the loads alive; practically never taken)
}

// ------------------------------------------------------------------ the NVFP4 encoder (ceiling scales)
// reference: quantize_nvfp4 in ScalesMode::Ceil, converter/src/main.rs:550-664 with encode_ue4m3_ceil / encode_subblock_ceil
// (:141-169, :404-410) and e2m1_index (:111-119): f32 values -> container blocks (4 scale bytes + 32 code bytes per 64
// values) and the tensor's global scale.  Every division the converter makes with `/` is a correctly rounded IEEE division
// here (raw = amax / 6, global = max raw / 448, r = raw / global, inv = 1 / dec); the codes are chosen against
// |v| * inv, the reciprocal, exactly as the converter does.
//
// The scale byte: the converter's search (start from floor(log2 r) + 7, step through mantissas with ceil, carry, then bump
// while the decoded byte is still below r) ends - whatever its log2 returns at a power of two - at the SMALLEST byte whose
// value is >= r, or 0x7F when r is beyond 480.  With r >= 2^-6 that byte is r's own f32 pattern rounded UP to three mantissa
// bits (exponent field e + 120, the mantissa's top three bits m); below, the subnormal ladder m = ceil(512 r).  r <= 0 gives
// 0, and the one NaN the arithmetic can make (inf / inf) the 0x38 the converter's casts make of it.
__device__ __forceinline__ unsigned ue4m3_ceil_byte(float r) {
    if (!(r == r)) return 0x38u;
    if (r <= 0.0f) return 0u;
    if (r > 480.0f) return 0x7Fu;
    if (r < 0x1p-6f) {
        const unsigned m = (unsigned)ceilf(r * 512.0f);  // 1..8 (exact product)
        return m;                                        // 8 = the first normal byte, 2^-6
    }
    unsigned u = __float_as_uint(r);
    if (u & 0xFFFFFu) u = (u | 0xFFFFFu) + 1u;
    return (((u >> 23) - 120u) << 3) | ((u >> 20) & 7u);
}
__device__ __forceinline__ float ue4m3_value(unsigned byte) {  // decode_ue4m3 (bytes 0..0x7F; 0x7F = 480)
    return __uint_as_float((byte & 0x7Fu) << 20) * 0x1p120f;
}
// the largest |v| of 16 values (f32::max ignores a NaN operand, like fmaxf), and the sub-block's raw scale: that over 6
__device__ __forceinline__ float subblock_amax(const float4 (&q)[4]) {
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) m = fmaxf(fmaxf(fmaxf(fmaxf(m, fabsf(q[i].x)), fabsf(q[i].y)), fabsf(q[i].z)), fabsf(q[i].w));
    return m;
}
__device__ __forceinline__ float subblock_raw(const float4 (&q)[4]) { return __fdiv_rn(subblock_amax(q), 6.0f); }
// pass 1: the largest |value| of the tensor, as the bit pattern of a non-negative f32 (they order like unsigned integers).
// The largest raw scale is that maximum over 6: a correctly rounded division is monotonic, so the maximum of the quotients is
// the quotient of the maximum, bit for bit.  Grid-stride over the n / 16 sub-blocks, one atomic per block; *max_bits starts
// as 0 (quantize_nvfp4_clear: a kernel rather than a memset, so that the three launches can be captured into a graph).
extern "C" __global__ void quantize_nvfp4_clear(unsigned* __restrict__ max_bits) { *max_bits = 0u; }
extern "C" __global__ void __launch_bounds__(256) quantize_nvfp4_amax(const float* __restrict__ values, unsigned long long n_sub,
                                                                       unsigned* __restrict__ max_bits) {
    __shared__ float per_wave[4];
    float best = 0.0f;
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < n_sub; i += (unsigned long long)gridDim.x * blockDim.x) {
        const float4* p = (const float4*)(values + 16 * i);
        const float4 q[4] = {p[0], p[1], p[2], p[3]};
        best = fmaxf(best, subblock_amax(q));
    }
    for (int o = 32; o > 0; o >>= 1) best = fmaxf(best, __shfl_xor(best, o));
    if ((threadIdx.x & 63u) == 0) per_wave[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        best = fmaxf(fmaxf(per_wave[0], per_wave[1]), fmaxf(per_wave[2], per_wave[3]));
        if (best > 0.0f) atomicMax(max_bits, __float_as_uint(best));
    }
}
// pass 2: one thread per sub-block: its scale byte and its sixteen codes; thread 0 also leaves the global scale
extern "C" __global__ void __launch_bounds__(256) quantize_nvfp4_encode(const float* __restrict__ values, unsigned long long n_sub,
                                                                         const unsigned* __restrict__ max_bits, unsigned char* __restrict__ blocks,
                                                                         float* __restrict__ global_out) {
    const float max_scale = __fdiv_rn(__uint_as_float(*max_bits), 6.0f);  // the largest raw scale (see pass 1)
    const float global = max_scale > 0.0f ? __fdiv_rn(max_scale, 448.0f) : 1.0f;
    const unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i == 0) global_out[0] = global;
    if (i >= n_sub) return;
    const float4* p = (const float4*)(values + 16 * i);
    const float4 q[4] = {p[0], p[1], p[2], p[3]};
    const unsigned byte = ue4m3_ceil_byte(__fdiv_rn(subblock_raw(q), global));
    const float dec = ue4m3_value(byte) * global;
    const float inv = __fdiv_rn(1.0f, dec);
    auto code = [&](float v) -> unsigned {
        const float m = fabsf(v) * inv;  // (0 * inf = NaN: every comparison false, code 0, as in the converter)
        const unsigned idx = (unsigned)(m >= 0.25f) + (unsigned)(m >= 0.75f) + (unsigned)(m >= 1.25f) + (unsigned)(m >= 1.75f) + (unsigned)(m >= 2.5f) +
                             (unsigned)(m >= 3.5f) + (unsigned)(m >= 5.0f);
        return idx | ((v < 0.0f) ? 8u : 0u);
    };
    unsigned lo = 0, hi = 0;  // values 0..7 and 8..15 of the sub-block, four bits each, value j in bits 4 j
#pragma unroll
    for (int k = 0; k < 2; k++) {
        lo |= (code(q[k].x) | (code(q[k].y) << 4) | (code(q[k].z) << 8) | (code(q[k].w) << 12)) << (16 * k);
        hi |= (code(q[2 + k].x) | (code(q[2 + k].y) << 4) | (code(q[2 + k].z) << 8) | (code(q[2 + k].w) << 12)) << (16 * k);
    }
    unsigned char* blk = blocks + (i >> 2) * CROW_BLOCK_BYTES;
    const unsigned sb = (unsigned)(i & 3);
    blk[sb] = (unsigned char)byte;
    unsigned* codes = (unsigned*)(blk + 4 + 8 * sb);  // (36-byte blocks: every code dword is four-byte aligned)
    codes[0] = lo;
    codes[1] = hi;
}

// ------------------------------------------------------------------ router
// Wave-wide maximum of an unsigned key through the data-parallel lane moves (an inclusive scan along the rows of 16
// lanes, then the two row broadcasts; lane 63 ends with the maximum): six dependent vector instructions where a
// butterfly of lane shuffles takes six round trips through the LDS crossbar.  All 64 lanes must be active.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ unsigned dpp_umax_step(unsigned v) {
    const unsigned o = (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
    return o > v ? o : v;
}
__device__ __forceinline__ unsigned wave_umax(unsigned v) {
    v = dpp_umax_step<0x111, 0xf>(v);  // row_shr:1
    v = dpp_umax_step<0x112, 0xf>(v);  // row_shr:2
    v = dpp_umax_step<0x114, 0xf>(v);  // row_shr:4
    v = dpp_umax_step<0x118, 0xf>(v);  // row_shr:8
    v = dpp_umax_step<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_umax_step<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
    return (unsigned)__builtin_amdgcn_readlane((int)v, 63);
}

// Wave-wide float maximum, the same lane moves as wave_umax (identity -inf); and the halving-tree sum in which lane t takes
// lane t + 32, then + 16 (the two half / quarter swaps), then + 8, 4, 2, 1 (row shifts): lane 0 ends with exactly the sum a
// shuffle-down tree gives, each step the same single f32 addition.  Both return the result in every lane.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_fmax_step(float v) {
    const float o = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, -INFINITY), __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
    return fmaxf(o, v);
}
__device__ __forceinline__ float wave_fmax(float v) {
    v = dpp_fmax_step<0x111, 0xf>(v);
    v = dpp_fmax_step<0x112, 0xf>(v);
    v = dpp_fmax_step<0x114, 0xf>(v);
    v = dpp_fmax_step<0x118, 0xf>(v);
    v = dpp_fmax_step<0x142, 0xa>(v);
    v = dpp_fmax_step<0x143, 0xc>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
template <int CTRL>
__device__ __forceinline__ float dpp_shl_add(float v) {  // lane t: v[t] + v[t + n] inside its row of 16 (row_shl:n); lanes without a source add 0
    const float o = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
    return __fadd_rn(v, o);
}
__device__ __forceinline__ float wave_tree_sum(float v) {
    const unsigned b = __float_as_uint(v);
    const u32x2 h = __builtin_amdgcn_permlane32_swap(b, b, false, false);  // .x = lanes 0..31's value, .y = lanes 32..63's
    v = __fadd_rn(__uint_as_float(h.x), __uint_as_float(h.y));
    const unsigned c = __float_as_uint(v);
    const u32x2 q = __builtin_amdgcn_permlane16_swap(c, c, false, false);  // .x = the even 16-lane group's value, .y = the odd one's
    v = __fadd_rn(__uint_as_float(q.x), __uint_as_float(q.y));
    v = dpp_shl_add<0x108>(v);
    v = dpp_shl_add<0x104>(v);
    v = dpp_shl_add<0x102>(v);
    v = dpp_shl_add<0x101>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
}

// One token's routing on one wavefront, SLOTS = E / 64 experts per lane: expert e lives in lane e % 64, slot e / 64.
template <int SLOTS>
__device__ __forceinline__ void router_body(const float* __restrict__ logits, const unsigned int* __restrict__ bitmap, int* __restrict__ ids,
                                            float* __restrict__ wts, unsigned long long* __restrict__ gu_ptrs,
                                            unsigned long long* __restrict__ dn_ptrs, const unsigned long long* __restrict__ table,
                                            unsigned int* __restrict__ cold_mask, unsigned long long* __restrict__ counters,
                                            unsigned long long* __restrict__ sel_counts, int K, int t, bool write, int& picked) {
    constexpr int E = SLOTS * 64;
    const int lane = lane_id();
    float l[SLOTS], red[SLOTS];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < SLOTS; j++) {
        l[j] = logits[(size_t)t * E + j * 64 + lane];
        mx = fmaxf(mx, l[j]);
    }
    mx = wave_fmax(mx);
#pragma unroll
    for (int j = 0; j < SLOTS; j++) red[j] = l[j] = expf(l[j] - mx);
    // tree over E slots: strides E/2 .. 64 pair slots inside a lane, strides 32 .. 1 pair lanes
#pragma unroll
    for (int st = SLOTS / 2; st > 0; st >>= 1)
#pragma unroll
        for (int j = 0; j < st; j++) red[j] += red[j + st];
    const float den = wave_tree_sum(red[0]);
    // keys: probabilities are >= 0, so their bit patterns order like the values; + 1 keeps 0 for "already picked"
    unsigned key[SLOTS];
#pragma unroll
    for (int j = 0; j < SLOTS; j++) key[j] = __float_as_uint(l[j] / den) + 1u;
    float sum = 0.0f, my_w = 0.0f;
    int my_id = 0;
    for (int k = 0; k < K; k++) {
        unsigned best = key[0];
        int best_id = lane;  // the lane's best: lowest slot (= lowest id in this lane) on ties
#pragma unroll
        for (int j = 1; j < SLOTS; j++)
            if (key[j] > best) {
                best = key[j];
                best_id = j * 64 + lane;
            }
        const unsigned top = wave_umax(best);
        const unsigned long long tied = __ballot(best == top);
        int pick;
        if (__popcll(tied) == 1) {
            pick = __builtin_amdgcn_readlane(best_id, (int)__builtin_ctzll(tied));
        } else {  // equal probabilities in several lanes: the lowest expert id
            const unsigned inv = best == top ? ~(unsigned)best_id : 0u;
            pick = (int)~wave_umax(inv);
        }
        const float pw = __uint_as_float(top - 1u);
        sum += pw;
        if (lane == k) {
            my_w = pw;
            my_id = pick;
        }
        if ((pick & 63) == lane) {
#pragma unroll
            for (int j = 0; j < SLOTS; j++)
                if (j == (pick >> 6)) key[j] = 0u;
        }
    }
    picked = my_id;  // lane k: the k-th pick
    if (!write) return;
    unsigned cold = 0;
    if (lane < K) {
        wts[(size_t)t * K + lane] = my_w / sum;
        ids[(size_t)t * K + lane] = my_id;
        if (table) {
            if (gu_ptrs) gu_ptrs[(size_t)t * K + lane] = table[my_id * 2];
            if (dn_ptrs) dn_ptrs[(size_t)t * K + lane] = table[my_id * 2 + 1];
        }
        if (sel_counts) atomicAdd(&sel_counts[my_id], 1ull);
        if (bitmap && !((bitmap[my_id >> 5] >> (my_id & 31)) & 1u)) cold = 1u << lane;
    }
    if (cold_mask || counters) {
        for (int o = 32; o > 0; o >>= 1) cold |= __shfl_xor(cold, o);
        if (lane == 0) {
            if (cold_mask) cold_mask[t] = cold;
            if (counters) {
                atomicAdd(&counters[0], (unsigned long long)K);
                atomicAdd(&counters[1], (unsigned long long)__popc(cold));
            }
        }
    }
}

__device__ __forceinline__ void router_dispatch(int E, const float* __restrict__ logits, const unsigned int* __restrict__ bitmap, int* __restrict__ ids,
                                                float* __restrict__ wts, unsigned long long* __restrict__ gu_ptrs, unsigned long long* __restrict__ dn_ptrs,
                                                const unsigned long long* __restrict__ table, unsigned int* __restrict__ cold_mask,
                                                unsigned long long* __restrict__ counters, unsigned long long* __restrict__ sel_counts, int K, int t,
                                                bool write, int& picked) {
    switch (E >> 6) {
        case 1: router_body<1>(logits, bitmap, ids, wts, gu_ptrs, dn_ptrs, table, cold_mask, counters, sel_counts, K, t, write, picked); break;
        case 2: router_body<2>(logits, bitmap, ids, wts, gu_ptrs, dn_ptrs, table, cold_mask, counters, sel_counts, K, t, write, picked); break;
        case 4: router_body<4>(logits, bitmap, ids, wts, gu_ptrs, dn_ptrs, table, cold_mask, counters, sel_counts, K, t, write, picked); break;
        case 8: router_body<8>(logits, bitmap, ids, wts, gu_ptrs, dn_ptrs, table, cold_mask, counters, sel_counts, K, t, write, picked); break;
        default: router_body<16>(logits, bitmap, ids, wts, gu_ptrs, dn_ptrs, table, cold_mask, counters, sel_counts, K, t, write, picked); break;
    }
}

// reference: router_top10, engine/src/kernels.rs:3109-3184.  grid (T), block 64: one wavefront per
// token.  The softmax denominator is added in the reference's halving-tree order (slots first, then
// lanes), so weights match an E-thread tree.  Ties go to the lowest expert id.
// E = model.experts (power of two, 64..1024), K = model.topk <= 16 (the geometry the launcher appends).
// bitmap / cold_mask / counters / sel_counts / table / *_ptrs may be null (skipped).
extern "C" __global__ void __launch_bounds__(64) router_top10(const float* __restrict__ logits, const unsigned int* __restrict__ bitmap,
                                                              int* __restrict__ ids, float* __restrict__ wts,
                                                              unsigned long long* __restrict__ gu_ptrs, unsigned long long* __restrict__ dn_ptrs,
                                                              const unsigned long long* __restrict__ table, unsigned int* __restrict__ cold_mask,
                                                              unsigned long long* __restrict__ counters, unsigned long long* __restrict__ sel_counts,
                                                              const Geo model) {
    const int E = model.experts, K = model.topk;
    if (E < 64 || E > 1024 || (E & (E - 1)) != 0 || K < 1 || K > 16 || K > E || block_threads() != 64) {
        if (threadIdx.x == 0) atomicOr(g_ws.status, STATUS_BAD_GEO);
        return;
    }
    int picked;
    router_dispatch(E, logits, bitmap, ids, wts, gu_ptrs, dn_ptrs, table, cold_mask, counters, sel_counts, K, (int)blockIdx.x, true, picked);
}

// Router and routed gate|up + SwiGLU in ONE launch: every block works out its token's routing itself (wave 0; the
// logits row is 1 KB) instead of reading pointers a router launch left behind, which takes a launch (4 us back to back) off
// the layer.  grid (inter / 16, 1, T K), block as moe_gate_up_silu.  Block (strip 0, pick 0) of each token writes
// ids, wts and dn_ptrs for moe_down_combine.  table[2 e] / table[2 e + 1] = gate|up / down slab of expert e.
extern "C" __global__ void __launch_bounds__(1024) moe_route_gate_up_silu(const float* __restrict__ logits, const unsigned long long* __restrict__ table,
                                                                          const float* __restrict__ x, const float* __restrict__ gs_ptr,
                                                                          float* __restrict__ h, int* __restrict__ ids, float* __restrict__ wts,
                                                                          unsigned long long* __restrict__ dn_ptrs, const int* __restrict__ k_dim_p,
                                                                          const int* __restrict__ x_stride_p, const int* __restrict__ inter_p, int geo, const Workspace ws,
                                                                          const Geo model) {
    ENTER(logits, table, x, gs_ptr, h, ids, wts, dn_ptrs, k_dim_p, x_stride_p, inter_p, geo);
    const int pairs = geo & 0xFFFFF;
    __shared__ unsigned long long s_slab;
    const int E = model.experts, K = model.topk;
    if (E < 64 || E > 1024 || (E & (E - 1)) != 0 || K < 1 || K > 16 || K > E || table == nullptr) {
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_GEO);
        return;
    }
    const int combo = (int)blockIdx.z, t = combo / K, j = combo % K;
    if (threadIdx.x < 64) {  // wave 0
        // Up to 256 experts the whole pointer table (16 bytes per expert) is requested together with the logits, four entries
        // per lane, and the picked expert's entry is taken from registers: read after the routing it would be one more
        // dependent round trip between the logits and the block's first weight load.
        const int lane = (int)threadIdx.x;
        u32x4 entry[4];
        if (E <= 256) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int i = lane + 64 * q;
                entry[q] = *(const __attribute__((address_space(1))) u32x4*)((const unsigned char*)table + 16 * (size_t)(i < E ? i : 0));
            }
        }
        int picked;
        router_dispatch(E, logits, nullptr, ids, wts, nullptr, dn_ptrs, table, nullptr, nullptr, nullptr, K, t, blockIdx.x == 0 && j == 0, picked);
        const int e = __builtin_amdgcn_readlane(picked, j);
        if (E <= 256) {
            const int q = e >> 6;  // uniform
            const u32x4 mine = q == 0 ? entry[0] : (q == 1 ? entry[1] : (q == 2 ? entry[2] : entry[3]));
            const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)mine.x, e & 63), hi = (unsigned)__builtin_amdgcn_readlane((int)mine.y, e & 63);
            if (threadIdx.x == 0) s_slab = ((unsigned long long)hi << 32) | lo;
        } else if (threadIdx.x == 0) {
            s_slab = table[2 * e];
        }
    }
    __syncthreads();
    const int inter = *inter_p;
    const unsigned char* w = (const unsigned char*)s_slab;
    CROW_REFUSE_NULL_SLAB(w);  // a table with an empty entry: uniform over the block, after the only barrier before the body
    if (inter % CROW_STRIP_ROWS != 0) {
        if (threadIdx.x == 0) atomicOr(ws.status, STATUS_BAD_SHAPE);
        return;
    }
    GemvArgs a = gemv_args(w, w + up_offset(inter, pairs), gs_ptr, gs_ptr, x + (size_t)t * *x_stride_p, 0, h, 0, pairs, k_dim_p, inter_p);
    a.y_row0 = combo;
    gemv_body<2, 1, false, EPI_SILU_GU>(a, blockIdx.z, LDS, ws);
}

// Sort the n routed combos of a batch by expert and cut them into tiles of at most four combos of one expert: the work of
// moe_count + moe_plan + moe_scatter (engine/src/kernels.rs:3334-3384) in ONE launch of one block (the reference needs
// three because its plan also schedules host-to-device staging of cold experts, which does not exist here; its tiles hold
// up to 8 combos, the width of its MMA; four is the row count of this library's GEMV).  ids[n] = expert of combo c;
// perm[n] = the combos in expert order, ascending combo inside an expert (stable, so the result does not depend on timing);
// tiles[t] = (expert, first position in perm, combos, 0), experts ascending; *n_tiles.
// A counting sort over chunks of 64 combos (one wavefront pass each): per-chunk histograms, a running sum per expert
// over the chunks, a block scan over the experts, then every chunk ranks its combos among equal experts with ballots.
// n <= 4096, E = model.experts <= 1024, E * ceil(n / 64) <= 16384.  grid 1, block 1024.
#define CROW_MOE_GROUP_MAX_COMBOS 4096
#define CROW_MOE_GROUP_HIST 16384
extern "C" __global__ void __launch_bounds__(1024) moe_group(const int* __restrict__ ids, const int* __restrict__ n_p, int* __restrict__ perm,
                                                             int4* __restrict__ tiles, int* __restrict__ n_tiles, const int* __restrict__ max_tiles_p,
                                                             const Geo model) {
    __shared__ unsigned short s_hist[CROW_MOE_GROUP_HIST];  // [chunk][expert]: count, then the count in earlier chunks
    __shared__ int s_off[1024], s_tile[1024];
    __shared__ int s_bad;
    const int n = *n_p, E = model.experts, max_tiles = *max_tiles_p, t = (int)threadIdx.x;
    const int chunks = (n + 63) >> 6;
    if (block_threads() != 1024 || n < 0 || n > CROW_MOE_GROUP_MAX_COMBOS || E < 1 || E > 1024 || E * chunks > CROW_MOE_GROUP_HIST) {
        if (t == 0) {
            atomicOr(g_ws.status, STATUS_BAD_GEO);
            *n_tiles = 0;
        }
        return;
    }
    for (int i = t; i < E * chunks; i += 1024) s_hist[i] = 0;
    if (t == 0) s_bad = 0;
    __syncthreads();
    // per-chunk histograms (16-bit counters, two to a word: add 1 or 1 << 16)
    for (int i = t; i < n; i += 1024) {
        const int e = ids[i];
        if (e < 0 || e >= E) s_bad = 1;
        else {
            const int slot = (i >> 6) * E + e;
            atomicAdd((unsigned*)s_hist + (slot >> 1), (slot & 1) ? 0x10000u : 1u);
        }
    }
    __syncthreads();
    if (s_bad) {  // an expert id outside the geometry: nothing is planned
        if (t == 0) {
            atomicOr(g_ws.status, STATUS_BAD_GEO);
            *n_tiles = 0;
        }
        return;
    }
    // thread = expert: counts of earlier chunks, and the expert's total
    int cnt = 0;
    if (t < E) {
        for (int c = 0; c < chunks; c++) {
            const int v = s_hist[c * E + t];
            s_hist[c * E + t] = (unsigned short)cnt;
            cnt += v;
        }
    }
    const int tc = (cnt + 3) >> 2;
    // inclusive scans over the experts - combos, and tiles of four - inside each wavefront by lane shifts, then over the
    // sixteen wavefronts' totals: two block barriers instead of two per doubling step
    const int ln = lane_id(), wv = t >> 6;
    int so = cnt, st = tc;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int a = __shfl_up(so, d), b = __shfl_up(st, d);
        if (ln >= d) {
            so += a;
            st += b;
        }
    }
    if (ln == 63) {
        s_off[wv] = so;
        s_tile[wv] = st;
    }
    __syncthreads();
    int base_o = 0, base_t = 0, total_tiles = 0;
#pragma unroll
    for (int q = 0; q < 16; q++) {
        const int a = s_off[q], b = s_tile[q];
        if (q < wv) {
            base_o += a;
            base_t += b;
        }
        total_tiles += b;
    }
    __syncthreads();  // the totals are read before s_off is reused below
    const int first = base_o + so - cnt, first_tile = base_t + st - tc;
    if (total_tiles > max_tiles) {  // uniform: every thread reads the same total
        if (t == 0) {
            atomicOr(g_ws.status, STATUS_WORKSPACE_TOO_SMALL);
            *n_tiles = 0;
        }
        return;
    }
    if (t == 0) *n_tiles = total_tiles;
    for (int q = 0; q < tc; q++) tiles[first_tile + q] = make_int4(t, first + 4 * q, cnt - 4 * q < 4 ? cnt - 4 * q : 4, 0);
    s_off[t] = first;  // now: the expert's first position in perm
    __syncthreads();
    // every chunk (one wavefront pass) ranks its combos among equal experts: position = expert's first + earlier chunks + rank
    const int lane = lane_id(), wave = t >> 6;
    for (int c = wave; c < chunks; c += 16) {
        const int i = c * 64 + lane;
        const bool live = i < n;
        const int e = live ? ids[i] : -1;
        int rank = 0;
        unsigned long long todo = __ballot(live);
        while (todo) {  // one round per distinct expert of the chunk
            const int lead = __builtin_amdgcn_readlane(e, (int)__builtin_ctzll(todo));
            const unsigned long long same = __ballot(e == lead);
            if (e == lead) rank = __popcll(same & ((1ull << lane) - 1ull));
            todo &= ~same;
        }
        if (live) perm[s_off[e] + s_hist[c * E + e] + rank] = i;
    }
}

// reference: silu_mul_combo, engine/src/kernels.rs:1562-1570: [C][2 I] -> [C][I], I = model.inter
extern "C" __global__ void silu_mul_combo(const float* __restrict__ h1, float* __restrict__ h2, const int* __restrict__ n_p, const Geo model) {
    const int i = (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (i >= *n_p) return;
    const int inter = model.inter;
    const int c = i / inter, j = i % inter;
    h2[i] = silu_mul(h1[(size_t)c * 2 * inter + j], h1[(size_t)c * 2 * inter + inter + j]);
}

// reference: acc_combo, engine/src/kernels.rs:1583-1592: y[t][c] += sum_j rw[t][j] * x[t K + j][c],
// j ascending, one rounding per multiply and per add.  grid (ceil(H / 256), T), block 256.
extern "C" __global__ void acc_combo(const float* __restrict__ x, const float* __restrict__ rw, float* __restrict__ y, const Geo model) {
    const int H = model.hidden, K = model.topk;
    const int c = (int)(blockIdx.x * blockDim.x + threadIdx.x), t = (int)blockIdx.y;
    if (c >= H) return;
    float acc = 0.0f;
    for (int j = 0; j < K; j++) {
        const float prod = rw[t * K + j] * x[((size_t)t * K + j) * H + c];
        acc = __fadd_rn(acc, prod);
    }
    y[(size_t)t * H + c] += acc;
}

// ------------------------------------------------------------------ greedy argmax
// (the order itself: device_common.h)
// grid (1), block up to 1024
extern "C" __global__ void __launch_bounds__(1024) argmax_k(const float* __restrict__ logits, int* __restrict__ out, const int* __restrict__ n_p) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const int n = *n_p;
    Best b{-3.0e38f, 0};
    for (int i = (int)threadIdx.x; i < n; i += (int)blockDim.x) {
        const float v = logits[i];
        if (better(v, i, b.v, b.i)) {
            b.v = v;
            b.i = i;
        }
    }
    b = wave_best(b);
    const int wave = (int)(threadIdx.x >> 6), waves = (int)((blockDim.x + 63) >> 6);
    if (lane_id() == 0) {
        sv[wave] = b.v;
        si[wave] = b.i;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < waves; w++)
            if (better(sv[w], si[w], b.v, b.i)) {
                b.v = sv[w];
                b.i = si[w];
            }
        out[0] = b.i;
    }
}

// The fused head's second kernel, started by the launcher right behind gemv_nvfp4_w_argmax (callers launch ONE kernel): the
// maximum of the `strips` keys the GEMV's blocks left in the head's scratch, decoded into the greedy token.  One block of 1024
// threads, every thread's loads in flight at once; the order is a total order on keys, so the reduction shape is free.
extern "C" __global__ void __launch_bounds__(1024) argmax_finish(int* __restrict__ out, unsigned strips, const Workspace ws) {
    __shared__ unsigned long long wave_max[16];
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    unsigned long long best = 0;
    for (unsigned base = threadIdx.x; base < strips; base += 16 * 1024) {  // sixteen loads in flight per thread: one round trip
        unsigned long long k[16];
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const unsigned i = base + 1024u * j;
            k[j] = ws.head[i < strips ? i : base];
        }
#pragma unroll
        for (int j = 0; j < 16; j++) best = k[j] > best ? k[j] : best;
    }
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = ((unsigned long long)__shfl_xor((unsigned)(best >> 32), o) << 32) | __shfl_xor((unsigned)best, o);
        best = other > best ? other : best;
    }
    if (lane == 0) wave_max[wave] = best;
    __syncthreads();
    if (threadIdx.x != 0) return;
    for (int w = 1; w < 16; w++) best = wave_max[w] > best ? wave_max[w] : best;
    out[0] = best != 0ull ? best_key_index(best) : 0;
}

// ------------------------------------------------------------------ BF16 and F32 keeps
// The tensors the container keeps unquantised (router, q/k, MTP head): y[t][row] = sum_k w[row][k] * x[t][k], f32
// activations, f32 accumulation.  16-byte non-temporal weight loads (8 bf16 or 4 f32 per lane per step: 1024 contiguous
// bytes per wave instruction), x through the vector cache (it is re-read by every row).  Two launch shapes, told apart by
// grid.x, block 256 in both:
//   grid (ceil(rows / 4), T)   one wavefront per (row, t): the shape for tall tensors (crow_hip_launch_dims picks it
//                              when rows * T > 2048)
//   grid (rows, T)             one block per (row, t), its four waves take every fourth 1024-byte run of the row and add
//                              their sums in wave order through LDS: a short tensor (the router: 256 rows) still puts a
//                              thousand waves on the chip, and a row's loads are all in flight at once.  This is also
//                              the grid of the reference's block-per-row kernels, whose call sites keep their dims.
// Order: a lane adds its products in column order with one FMA each, four steps of loads in flight at a time, then the
// 64 lane sums are added by halving (lane l += lane l + 32, + 16, ... + 1), then (second shape) the wave sums in wave order.
//   gemv_bf16_w   engine/src/kernels.rs:1130-1157 (warp per row; k_dim % 8 == 0)
//   gemv_bf16     engine/src/kernels.rs:1061-1077 (block per row, one token; + rows_p: the reference's grid.x is the row count)
//   gemv_bf16_b   engine/src/kernels.rs:1080-1098 (block per row, grid.y tokens; + rows_p)
//   gemv_b        engine/src/kernels.rs:97-115   (f32 weights, the router projection of gen.rs:4182; + rows_p; k_dim % 4 == 0)
//   gemv_bf16_ws  engine/src/kernels.rs:1430-1458 (gemv_bf16_w with y = 1 / (1 + expf(-sum)) at the store)
//   gemv_bf16_bs  engine/src/kernels.rs:1100-1124 (gemv_bf16_b with an explicit y row stride; + rows_p)
template <bool WBF16, bool SIGMOID = false>
__device__ __forceinline__ void keep_gemv_body(const void* __restrict__ w, const float* __restrict__ x, float* __restrict__ y, int k, int rows,
                                               size_t y_stride) {
    constexpr int PER = WBF16 ? 8 : 4;  // weights per 16-byte load
    __shared__ float wave_sum[4];
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = lane_id();
    const bool block_per_row = gridDim.x == (unsigned)rows;  // uniform over the launch
    const int row = block_per_row ? (int)blockIdx.x : (int)blockIdx.x * 4 + wave, t = (int)blockIdx.y;
    if (row >= rows) return;  // (first shape only: a whole wave leaves, nobody waits for it)
    const int parts = block_per_row ? 4 : 1, part = block_per_row ? wave : 0;
    const char* wp = (const char*)w + (size_t)row * k * (WBF16 ? 2 : 4);
    const float* xp = x + (size_t)t * k;
    const int run = parts * 64 * PER;  // columns between two loads of a lane
    float acc = 0.0f;
    for (int i0 = (part * 64 + lane) * PER; i0 < k; i0 += 4 * run) {
        uint4 v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = i0 + j * run;
            v[j] = make_uint4(0, 0, 0, 0);
            if (i < k) v[j] = stream_load((const uint4*)(wp + (size_t)i * (WBF16 ? 2 : 4)));
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int i = i0 + j * run;
            if (i < k) {
                const float4 a = *(const float4*)(xp + i);
                if (WBF16) {
                    const float4 b = *(const float4*)(xp + i + 4);
                    acc = __builtin_fmaf(__uint_as_float(v[j].x << 16), a.x, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].x & 0xffff0000u), a.y, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].y << 16), a.z, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].y & 0xffff0000u), a.w, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].z << 16), b.x, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].z & 0xffff0000u), b.y, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].w << 16), b.z, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].w & 0xffff0000u), b.w, acc);
                } else {
                    acc = __builtin_fmaf(__uint_as_float(v[j].x), a.x, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].y), a.y, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].z), a.z, acc);
                    acc = __builtin_fmaf(__uint_as_float(v[j].w), a.w, acc);
                }
            }
        }
    }
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o);
    auto finish = [](float v) { return SIGMOID ? 1.0f / (1.0f + expf(-v)) : v; };
    if (!block_per_row) {
        if (lane == 0) y[(size_t)t * y_stride + row] = finish(acc);
        return;
    }
    if (lane == 0) wave_sum[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) y[(size_t)t * y_stride + row] = finish(((wave_sum[0] + wave_sum[1]) + wave_sum[2]) + wave_sum[3]);
}
#define CROW_KEEP_GEMV(NAME, WT, WBF16)                                                                                              \
    extern "C" __global__ void __launch_bounds__(256) NAME(const WT* __restrict__ w, const float* __restrict__ x, float* __restrict__ y, \
                                                           const int* __restrict__ k_dim_p, const int* __restrict__ rows_p) {        \
        if (block_threads() != 256) {                                                                                                \
            if (threadIdx.x == 0) atomicOr(g_ws.status, STATUS_BAD_SHAPE);                                                           \
            return;                                                                                                                  \
        }                                                                                                                            \
        keep_gemv_body<WBF16>(w, x, y, *k_dim_p, *rows_p, (size_t)*rows_p);                                                          \
    }
CROW_KEEP_GEMV(gemv_bf16_w, unsigned short, true)
CROW_KEEP_GEMV(gemv_bf16, unsigned short, true)
CROW_KEEP_GEMV(gemv_bf16_b, unsigned short, true)
CROW_KEEP_GEMV(gemv_b, float, false)

extern "C" __global__ void __launch_bounds__(256) gemv_bf16_ws(const unsigned short* __restrict__ w, const float* __restrict__ x, float* __restrict__ y,
                                                               const int* __restrict__ k_dim_p, const int* __restrict__ rows_p) {
    if (block_threads() != 256) {
        if (threadIdx.x == 0) atomicOr(g_ws.status, STATUS_BAD_SHAPE);
        return;
    }
    keep_gemv_body<true, true>(w, x, y, *k_dim_p, *rows_p, (size_t)*rows_p);
}
extern "C" __global__ void __launch_bounds__(256) gemv_bf16_bs(const unsigned short* __restrict__ w, const float* __restrict__ x, float* __restrict__ y,
                                                               const int* __restrict__ k_dim_p, const int* __restrict__ y_stride_p,
                                                               const int* __restrict__ rows_p) {
    if (block_threads() != 256 || *y_stride_p < *rows_p) {
        if (threadIdx.x == 0) atomicOr(g_ws.status, STATUS_BAD_SHAPE);
        return;
    }
    keep_gemv_body<true>(w, x, y, *k_dim_p, *rows_p, (size_t)*y_stride_p);
}

// ------------------------------------------------------------------ measurement only: the one-row GEMV without matrix instructions
// The reference's own shape for this product (kernels_p2.rs:304-368: a warp per few rows, lanes across the columns, f32
// multiply-adds on decoded weights, a shuffle tree) written for 64-wide waves, on the CONTAINER layout as it stands (no repack),
// so that the choice of the matrix cores for one activation row rests on a measured number.  Not part of the drop-in set:
// the engine never asks for it.  Each 16-lane group of a wave owns RG adjacent rows and its lanes take every 16th 64-value
// block of them: per block and row one scale dword + eight code dwords, 32 conversions, 64 multiply-adds against the 64
// activations the lane holds for all its rows, one scale multiply-add per 16 values.  grid (ceil(rows / (16 RG))), block 256.
template <int RG>
__device__ __forceinline__ void gemv_valu_body(const unsigned char* __restrict__ w, const float* __restrict__ x, const float* __restrict__ gs_ptr,
                                               float* __restrict__ y, int k_dim, int rows) {
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    const int nb = k_dim / CROW_BLOCK_VALUES;
    const int row0 = (((int)blockIdx.x * 4 + wave) * 4 + (lane >> 4)) * RG, j = lane & 15;
    float acc[RG];
#pragma unroll
    for (int r = 0; r < RG; r++) acc[r] = 0.0f;
    for (int b = j; b < nb; b += 16) {
        f32x4 xv[16];
#pragma unroll
        for (int i = 0; i < 16; i++) xv[i] = *(const f32x4*)(x + (size_t)b * 64 + 4 * i);
#pragma unroll
        for (int r = 0; r < RG; r++) {
            const int row = row0 + r < rows ? row0 + r : rows - 1;
            const unsigned* blk = (const unsigned*)(w + ((size_t)row * nb + b) * CROW_BLOCK_BYTES);
            // the scale rule on four bytes at once: bit 7 cleared, 0x7F -> 0x7E
            unsigned sc = stream_load_u32(blk) & 0x7F7F7F7Fu;
            sc -= ((sc + 0x01010101u) & 0x80808080u) >> 7;
            unsigned c[8];
#pragma unroll
            for (int i = 0; i < 8; i++) c[i] = stream_load_u32(blk + 1 + i);
#pragma unroll
            for (int sb = 0; sb < 4; sb++) {
                float part = 0.0f;
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const unsigned cw = c[2 * sb + h];
                    const f32x2 v0 = fp4x2_to_f32<0>(cw), v1 = fp4x2_to_f32<1>(cw), v2 = fp4x2_to_f32<2>(cw), v3 = fp4x2_to_f32<3>(cw);
                    const f32x4 xa = xv[4 * sb + 2 * h], xb = xv[4 * sb + 2 * h + 1];
                    part = __builtin_fmaf(v0.x, xa.x, part);
                    part = __builtin_fmaf(v0.y, xa.y, part);
                    part = __builtin_fmaf(v1.x, xa.z, part);
                    part = __builtin_fmaf(v1.y, xa.w, part);
                    part = __builtin_fmaf(v2.x, xb.x, part);
                    part = __builtin_fmaf(v2.y, xb.y, part);
                    part = __builtin_fmaf(v3.x, xb.z, part);
                    part = __builtin_fmaf(v3.y, xb.w, part);
                }
                const float sv = sb == 0 ? e4m3_to_f32<0>(sc) : (sb == 1 ? e4m3_to_f32<1>(sc) : (sb == 2 ? e4m3_to_f32<2>(sc) : e4m3_to_f32<3>(sc)));
                acc[r] = __builtin_fmaf(part, sv, acc[r]);
            }
        }
    }
    const float gs = gs_ptr[0];
#pragma unroll
    for (int r = 0; r < RG; r++) {
        float v = acc[r];
        for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o);
        if (j == 0 && row0 + r < rows) y[row0 + r] = v * gs;
    }
}
#define CROW_VALU_ENTRY(NAME, RG)                                                                                                          \
    extern "C" __global__ void __launch_bounds__(256) NAME(const unsigned char* __restrict__ w, const float* __restrict__ x,              \
                                                           const float* __restrict__ gs_ptr, float* __restrict__ y,                       \
                                                           const int* __restrict__ k_dim_p, const int* __restrict__ rows_p) {             \
        const int k = *k_dim_p;                                                                                                            \
        if (block_threads() != 256 || k <= 0 || k % CROW_BLOCK_VALUES != 0) {                                                              \
            if (threadIdx.x == 0) atomicOr(g_ws.status, STATUS_BAD_SHAPE);                                                                 \
            return;                                                                                                                        \
        }                                                                                                                                  \
        gemv_valu_body<RG>(w, x, gs_ptr, y, k, *rows_p);                                                                                   \
    }
CROW_VALU_ENTRY(gemv_nvfp4_w_valu1, 1)
CROW_VALU_ENTRY(gemv_nvfp4_w_valu2, 2)
CROW_VALU_ENTRY(gemv_nvfp4_w_valu4, 4)

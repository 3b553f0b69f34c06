// Device-side state and helpers shared by every kernel of the library (one translation unit).
#pragma once
#include <hip/hip_runtime.h>
#include "layout.h"

namespace crow {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned stream_u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// blockDim.x read as a scalar from the kernel's implicit arguments (u16 group_size_x at byte 12 of the hidden block:
// the compiler's own blockDim.x is a 16-bit VECTOR load followed by a wait, which sits in front of the first weight
// load of every wave).  Launches here never have a partial last block, so the remainder field is not consulted.
__device__ __forceinline__ int block_threads() {
    const unsigned* ia = (const unsigned*)__builtin_amdgcn_implicitarg_ptr();
    return (int)(ia[3] & 0xffffu);
}

// 16-byte load of weight bytes that are read exactly once per launch: the non-temporal hint keeps them from
// displacing reusable lines in L2 and the memory-side cache (measured on a pure read of the tile pattern:
// 6.8-6.9 TB/s against 6.1-6.3 TB/s without the hint at 437 MB, 5.8 against 5.5 at 50 MB)
__device__ __forceinline__ uint4 stream_load(const uint4* p) {
    // weights are device memory: the explicit address space keeps the load a global one when `p` comes out of a select
    const stream_u32x4 v = __builtin_nontemporal_load((const __attribute__((address_space(1))) stream_u32x4*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ u32x4 stream_load_v(const uint4* p) {
    return __builtin_nontemporal_load((const __attribute__((address_space(1))) u32x4*)p);
}
// the same for one dword per lane (the scale words of a 256-column group)
__device__ __forceinline__ unsigned stream_load_u32(const unsigned* p) {
    return __builtin_nontemporal_load((const __attribute__((address_space(1))) unsigned*)p);
}

// Library-owned scratch for kernels that split one output tile over several workgroups:
// per-slice partial sums and one arrival counter per output tile.  Set once by crow_hip_init.
// Scratch of the fused head (gemv_nvfp4_w_argmax): one 64-bit key per 16-row strip.  Every block stores the best_key of its
// strip (a plain store: nobody reads it inside the launch), and the one-block kernel that the launcher starts right behind
// it (argmax_finish) takes the maximum.  Every launch overwrites the words it reads, so nothing is ever cleared.
struct Workspace {
    float* partials;
    unsigned* counters;
    unsigned long long partial_floats;  // capacity of `partials`
    unsigned counter_slots;             // capacity of `counters`
    unsigned* status;                   // device word: non-zero = a launch did not fit the workspace
    unsigned long long* head;           // fused lm_head argmax: one key per strip
    unsigned head_words;                // how many strips the head's scratch takes
};
__device__ Workspace g_ws;

// Model geometry the reference bakes into its kernel text as CN_* defines (engine/src/kernels.rs:5040-5125).  Here the
// kernels that need it take it BY VALUE as their last argument, which callers never pass: the launcher appends what
// crow_hip_set_geo last recorded on the host.  No device-side state, so setting it needs no copy and no synchronisation, and
// a launch captured into a graph keeps the geometry it was captured with.
struct Geo {
    int experts, topk, hidden, inter;
};

enum StatusBits : unsigned { STATUS_WORKSPACE_TOO_SMALL = 1u, STATUS_BAD_SHAPE = 2u, STATUS_BAD_GEO = 4u };

__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63u); }

// E2M1 pair decode: byte `SEL` of `word` holds two codes (low nibble first); the gfx950
// conversion instruction returns them as two exact f32 values (scale operand 1.0).
template <int SEL>
__device__ __forceinline__ f32x2 fp4x2_to_f32(unsigned word) {
    return __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, SEL);
}
template <int SEL>
__device__ __forceinline__ bf16x2 fp4x2_to_bf16(unsigned word) {
    return __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, SEL);
}
// UE4M3 scale decode of byte `SEL` (canonical bytes 0x00..0x7E only: OCP E4M3, exact)
template <int SEL>
__device__ __forceinline__ float e4m3_to_f32(unsigned word) {
    return __builtin_amdgcn_cvt_f32_fp8((int)word, SEL);
}

__device__ __forceinline__ unsigned u4_get(const uint4& v, int i) { return i == 0 ? v.x : (i == 1 ? v.y : (i == 2 ? v.z : v.w)); }

// silu(g) * u exactly as the reference kernels write it (kernels_p2.rs:386-387)
__device__ __forceinline__ float silu_mul(float g, float u) { return (g / (1.0f + expf(-g))) * u; }

// Greedy argmax order.  The reference (engine/src/kernels.rs:4238-4260) scans with 1024 strided
// threads (strict >, so a thread keeps its smallest index) and then halves a 1024-slot tree with
// strides 512 .. 1 in which slot t takes slot t + stride only when strictly greater.  Among equal
// maxima that tournament prefers bit 0 of t clear (the last round), then bit 1, ... : the winner is
// the position with the smallest BIT-REVERSED (i mod 1024), then the smallest i.  That is a total
// order, so any reduction shape gives the same index.  Start value -3.0e38 with index 0, as the
// reference.
struct Best {
    float v;
    int i;
};
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
    const unsigned ki = __brev((unsigned)i & 1023u), kb = __brev((unsigned)bi & 1023u);
    return v > bv || (v == bv && (ki < kb || (ki == kb && i < bi)));
}
// The same order as ONE unsigned 57-bit key, larger = better: the value's bits made monotonic (sign flipped for positive
// floats, all bits for negative ones; -0 counts as +0 and a NaN as the start value, as under the comparisons above) above
// the 25-bit complement of (bit-reversed (i mod 1024), i / 1024), i < 2^25.  A maximum over such keys is the tournament,
// whatever the arrival order.  No key of a real candidate is 0.
__device__ __forceinline__ unsigned long long best_key(float v, int i) {
    v = v == v ? v + 0.0f : -3.0e38f;
    const unsigned u = __float_as_uint(v);
    const unsigned hi = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    const unsigned tie = ((__brev((unsigned)i & 1023u) >> 22) << 15) | (((unsigned)i >> 10) & 0x7FFFu);
    return ((unsigned long long)hi << 25) | (unsigned long long)(0x1FFFFFFu - tie);
}
__device__ __forceinline__ int best_key_index(unsigned long long key) {
    const unsigned tie = 0x1FFFFFFu - (unsigned)(key & 0x1FFFFFFull);
    return (int)(((tie & 0x7FFFu) << 10) | (__brev(tie >> 15) >> 22));
}
__device__ __forceinline__ Best wave_best(Best b) {
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(b.v, o);
        const int oi = __shfl_xor(b.i, o);
        if (better(ov, oi, b.v, b.i)) {
            b.v = ov;
            b.i = oi;
        }
    }
    return b;
}

}  // namespace crow

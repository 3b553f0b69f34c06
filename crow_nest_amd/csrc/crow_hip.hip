// libcrow_hip.so: gfx950 code objects (built ahead of time from the headers below) and the C ABI
// declared in include/crow_hip.h.  One translation unit, so the device globals are shared.
#include <hip/hip_runtime.h>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/crow_hip.h"
#include "../../include/crow_hip_bench.h"
#include "kernels.h"
#include "misc_kernels.h"
#include "gemm.h"

namespace {

struct FnEntry {
    const char* name;
    const void* stub;
    int nargs;
    unsigned lds_fixed;  // dynamic LDS of a launch (kernels outside the GEMV family)
    // GEMV family (gemv.h): tensors per block (0 = not of the family), and the dynamic LDS of a block: the zero area + one
    // staging area per wave
    int nr;
    int max_waves;  // per block (the kernel's launch bound)
    int lds_per_wave;
    int ns;  // adjacent 16-row strips per block (kernels for several activation rows: CROW_MULTI_STRIPS), else 1
    bool takes_ws;  // the launcher appends the scratch descriptor (every kernel of the GEMV family)
    // a twin of `stub` for strips of two to eight groups that one wave walks alone, started in its place when the launch
    // dimensions say so; its dynamic LDS is the zero area and one staging area of twelve rows per GROUP (per block, not per wave)
    const void* tile_stub;
    bool takes_geo;  // the launcher appends the model geometry (crow_hip_set_geo) by value, last
};

// The launcher builds a kernel's argument array from the fields of its table entry: the caller's `nargs` values, then the
// geometry word (GEMV family), the scratch descriptor (takes_ws), the model geometry (takes_geo).  A kernel that gains a
// parameter its entry does not append would make HIP read an argument slot nobody wrote; the table is therefore checked
// against the kernels' own signatures when this file is compiled.
#define CROW_MAX_LAUNCH_ARGS 18
template <typename F>
struct arity;
template <typename... A>
struct arity<void (*)(A...)> {
    static constexpr int value = (int)sizeof...(A);
};
template <int NARGS, int APPENDED, typename F>
constexpr int checked_nargs(F) {
    static_assert(arity<F>::value == NARGS + APPENDED, "a kernel's parameter list and its table entry disagree");
    static_assert(NARGS + APPENDED <= CROW_MAX_LAUNCH_ARGS, "the launcher's argument array is too short for this kernel");
    return NARGS;
}
#define CROW_FN(name, nargs) {#name, (const void*)&name, checked_nargs<nargs, 0>(&name), 0u, 0, 16, 0, 1, false, nullptr, false}
#define CROW_FN_GEO(name, nargs) {#name, (const void*)&name, checked_nargs<nargs, 1>(&name), 0u, 0, 16, 0, 1, false, nullptr, true}
// NR tensors per block, bodies for 1 .. MMAX activation rows, bf16 or f32 activations
// (the bodies for several rows need more registers than a block of sixteen waves leaves each: they run in blocks of eight)
#define CROW_GEMV(name, nargs, NR, MMAX, XBF16) \
    {#name, (const void*)&name, checked_nargs<nargs, 2>(&name), 0u, NR, MMAX > 1 ? 8 : 16, crow::crow_gemv_lds_per_wave(MMAX, XBF16), MMAX > 1 ? (XBF16 ? CROW_MULTI_STRIPS_BF16 : CROW_MULTI_STRIPS) : 1, true, nullptr, false}
#define CROW_GEMV_GEO(name, nargs, NR, MMAX, XBF16) \
    {#name, (const void*)&name, checked_nargs<nargs, 3>(&name), 0u, NR, 16, crow::crow_gemv_lds_per_wave(MMAX, XBF16), 1, true, nullptr, true}
const FnEntry g_table[] = {
    CROW_GEMV(gemv_nvfp4_w, 6, 1, 1, false),       CROW_GEMV(gemv_nvfp4_w_bf16, 6, 1, 1, true),  CROW_GEMV(gemv_nvfp4_w_argmax, 7, 1, 1, false),
    CROW_GEMV(gemv_nvfp4_gu, 8, 2, 1, false),      CROW_GEMV(gemv_nvfp4_gu_bf16, 8, 2, 1, true),
    CROW_GEMV(gemv_nvfp4_wm, 7, 1, 4, false),      CROW_GEMV(gemv_nvfp4_gum, 9, 2, 4, false),
    CROW_GEMV(gemv_nvfp4_wm_bf16, 7, 1, 4, true),  CROW_GEMV(gemv_nvfp4_gum_bf16, 9, 2, 4, true), CROW_GEMV(gemv_fp4, 6, 1, 1, false),
    CROW_GEMV(gemv_fp4_b, 7, 1, 4, false),         CROW_GEMV(gemv_fp4_b1k, 7, 1, 4, false),      CROW_GEMV(gemv_fp4_bs, 8, 1, 4, false),
    CROW_GEMV(gemv_fp4_ptrb, 8, 1, 1, false),      CROW_GEMV(moe_gate_up_silu, 8, 2, 1, false),  CROW_GEMV_GEO(moe_down_combine, 7, 1, 1, false),
    CROW_GEMV_GEO(moe_route_gate_up_silu, 11, 2, 1, false),
    {"moe_gate_up_silu_grouped", (const void*)&moe_gate_up_silu_grouped, checked_nargs<11, 2>(&moe_gate_up_silu_grouped) + 0 * checked_nargs<11, 2>(&moe_gate_up_silu_grouped_tile), 0u, 2, 8, crow::crow_gemv_lds_per_wave(4, false), CROW_MULTI_STRIPS, true, (const void*)&moe_gate_up_silu_grouped_tile, false},
    {"moe_down_grouped", (const void*)&moe_down_grouped, checked_nargs<9, 2>(&moe_down_grouped) + 0 * checked_nargs<9, 2>(&moe_down_grouped_tile), 0u, 1, 8, crow::crow_gemv_lds_per_wave(4, false), CROW_MULTI_STRIPS, true, (const void*)&moe_down_grouped_tile, false},
    CROW_FN_GEO(moe_group, 6),
    CROW_FN_GEO(router_top10, 10), CROW_FN_GEO(silu_mul_combo, 3),  CROW_FN_GEO(acc_combo, 3),
    CROW_FN(argmax_k, 3),          CROW_FN(dequant_fp4_flat, 4),    CROW_FN(repack_nvfp4, 4),
    CROW_FN(unpack_nvfp4, 4),      CROW_FN(dequant_nvfp4_tiled, 5),
    // shared-X GEMM blocks: two staged X tiles of MT rows x 528 bytes
    {"gemm_nvfp4_bf16", (const void*)&gemm_nvfp4_bf16, checked_nargs<7, 0>(&gemm_nvfp4_bf16), 2u * 128u * 528u, 0, 16, 0, 1, false},
    {"gemm_nvfp4_bf16_m64", (const void*)&gemm_nvfp4_bf16_m64, checked_nargs<7, 0>(&gemm_nvfp4_bf16_m64), 2u * 64u * 528u, 0, 16, 0, 1, false},
    {"gemm_nvfp4_bf16_m48", (const void*)&gemm_nvfp4_bf16_m48, checked_nargs<7, 0>(&gemm_nvfp4_bf16_m48), 2u * 48u * 528u, 0, 16, 0, 1, false},
    {"gemm_nvfp4_bf16_m96", (const void*)&gemm_nvfp4_bf16_m96, checked_nargs<7, 0>(&gemm_nvfp4_bf16_m96), 2u * 96u * 528u, 0, 16, 0, 1, false},
    {"gemm_nvfp4_bf16_w48", (const void*)&gemm_nvfp4_bf16_w48, checked_nargs<7, 0>(&gemm_nvfp4_bf16_w48), 2u * 48u * 528u, 0, 8, 0, 1, false},
    {"gemm_nvfp4_bf16_w64", (const void*)&gemm_nvfp4_bf16_w64, checked_nargs<7, 0>(&gemm_nvfp4_bf16_w64), 2u * 64u * 528u, 0, 8, 0, 1, false},
    {"gemm_nvfp4_bf16_w80", (const void*)&gemm_nvfp4_bf16_w80, checked_nargs<7, 0>(&gemm_nvfp4_bf16_w80), 2u * 80u * 528u, 0, 8, 0, 1, false},
    {"gemm_nvfp4_bf16_w96", (const void*)&gemm_nvfp4_bf16_w96, checked_nargs<7, 0>(&gemm_nvfp4_bf16_w96), 2u * 96u * 528u, 0, 8, 0, 1, false},
    CROW_FN(gemm_nvfp4_bf16_m32, 7), CROW_FN(gemm_nvfp4_bf16_m16, 7), CROW_FN(gemv_bf16_w, 5),
    CROW_FN(gemv_bf16, 5), CROW_FN(gemv_bf16_b, 5), CROW_FN(gemv_b, 5), CROW_FN(gemv_bf16_ws, 5), CROW_FN(gemv_bf16_bs, 6),
    CROW_FN(gemv_nvfp4_w_valu1, 6), CROW_FN(gemv_nvfp4_w_valu2, 6), CROW_FN(gemv_nvfp4_w_valu4, 6),  // measurement only
};
const int g_table_n = (int)(sizeof(g_table) / sizeof(g_table[0]));

struct State {
    bool ready = false;
    int device = -1;
    int cus = 256;
    hipStream_t stream = nullptr;
    crow::Workspace ws{};
    crow::Workspace ws_static{};  // the same roles inside `scratch`, through the device address crow_hip_init asked for
    int* scalars = nullptr;  // device words for the library's own launches: (rows, k_dim) of the layout calls, the encoder's maxima
    char name[256] = {0};
    crow::Geo model{0, 0, 0, 0};  // the routed geometry (crow_hip_set_geo): appended by value to the kernels that take it
    size_t lds_cap = 64u * 1024u;  // most LDS one workgroup may take on this device
} g;

// Scratch memory of crow_hip_launch_noalloc: part of the code object, so it exists on a device from the moment the library
// is loaded there until the process ends, and no call ever allocates it.  Words [0, NOALLOC_PARTIAL_FLOATS) hold the partial
// sums of split launches, then NOALLOC_COUNTER_SLOTS arrival counters, the status word (alone on 32 words), and the fused
// head's keys (8 bytes per strip).
const unsigned HEAD_WORDS = 65536;  // the allocated workspace: heads of up to 1,048,576 rows
const unsigned NOALLOC_HEAD_WORDS = CROW_NOALLOC_MAX_HEAD_STRIPS;
const unsigned NOALLOC_PARTIAL_FLOATS = CROW_NOALLOC_MAX_PARTIAL_FLOATS;  // 4 MiB of split-K partial sums
const unsigned NOALLOC_COUNTER_SLOTS = CROW_NOALLOC_MAX_STRIPS;
const unsigned NOALLOC_TAIL_WORDS = 32 + 2 * NOALLOC_HEAD_WORDS;  // status line, then the head's 8-byte words
const unsigned NOALLOC_WORDS = NOALLOC_PARTIAL_FLOATS + NOALLOC_COUNTER_SLOTS + NOALLOC_TAIL_WORDS;
static __device__ __align__(256) unsigned scratch[NOALLOC_WORDS];
static_assert(sizeof(unsigned) * NOALLOC_WORDS == CROW_NOALLOC_SCRATCH_BYTES, "the header states the array's size");

const unsigned long long PARTIAL_FLOATS = 16ull << 20;  // 64 MiB of split-K partial sums
const unsigned COUNTER_SLOTS = 1u << 16;
// tile counters, then the status word
const unsigned COUNTER_WORDS = COUNTER_SLOTS + 1;

int hip_rc(hipError_t e) { return e == hipSuccess ? CROW_OK : (int)e; }

const FnEntry* find(const char* name) {
    if (!name) return nullptr;
    for (int i = 0; i < g_table_n; i++)
        if (strcmp(g_table[i].name, name) == 0) return &g_table[i];
    return nullptr;
}

// a handle is the address of a table entry, nothing else
const FnEntry* entry_of(crow_fn_t f) {
    const FnEntry* e = (const FnEntry*)(void*)f;
    if (e < g_table || e >= g_table + g_table_n) return nullptr;
    if (((const char*)e - (const char*)g_table) % (ptrdiff_t)sizeof(FnEntry) != 0) return nullptr;
    return e;
}


// Groups per strip if the grouped expert kernels take their twin for K / 64 = pairs (strips of two to eight groups that one
// wave walks alone in the launch shapes chosen below: up to 7 groups for one tensor, 10 - here 8 - per tensor for two), else 0.
unsigned tile_groups(int nr, unsigned pairs) {
    const unsigned groups = (pairs + CROW_GROUP_PAIRS - 1) / CROW_GROUP_PAIRS;
    return groups >= 2 && groups <= (nr == 2 ? (unsigned)CROW_TILE_MAX_GROUPS : 7u) ? groups : 0u;
}

// The launch dimensions of the GEMV family carry the problem in `gy` (crow_hip_launch_dims writes it, callers pass it on
// unchanged): bits 0..19 = K / 64, bits 20..23 = activation rows of the last token group (0 = not given), bits 24..31 = S, the
// number of column slices per strip.  The real grid is (gx, S, gz); the low 24 bits reach the kernel by value.
// `ws`: the scratch memory the launch may use, handed by value to the kernels that take one.
int launch_entry(const FnEntry* e, dim3 grid, dim3 block, const uint64_t* vals, uint32_t n, hipStream_t s, const crow::Workspace& ws) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!e || !vals) return CROW_ERR_BAD_ARGUMENT;
    if ((int)n != e->nargs) return CROW_ERR_ARG_COUNT;
    // whole wavefronts only: every kernel derives its wave count (and its LDS layout) from block.x / 64
    if (grid.x == 0 || grid.y == 0 || grid.z == 0 || block.x == 0 || block.x > 64u * (unsigned)e->max_waves || block.x % 64 != 0) return CROW_ERR_BAD_ARGUMENT;
    void* args[CROW_MAX_LAUNCH_ARGS];
    for (uint32_t i = 0; i < n; i++) args[i] = (void*)&vals[i];
    uint32_t na = n;
    size_t lds = e->lds_fixed;
    int geo = 0;
    crow::Workspace ws_arg = ws;
    const void* stub = e->stub;
    if (e->nr != 0) {
        const unsigned word = grid.y;
        const int pairs = (int)(word & 0xFFFFFu);
        const int waves = (int)(block.x / 64), wpt = waves / e->nr;
        if (pairs == 0 || wpt == 0) return CROW_ERR_BAD_ARGUMENT;
        if (e->tile_stub != nullptr && tile_groups(e->nr, (unsigned)pairs) != 0 && block.x <= 512) {
            // the twin for strips that one wave walks alone: strips per wave ride where S sits (such a strip is never cut into
            // slices), and the kernel takes the whole word; one staging area per group and block
            if ((word >> 24) == 0) return CROW_ERR_BAD_ARGUMENT;
            stub = e->tile_stub;
            geo = (int)word;
            grid.y = 1;
            lds = (size_t)CROW_GEMV_ZERO_BYTES + (size_t)tile_groups(e->nr, (unsigned)pairs) * (size_t)(e->lds_per_wave / 2);
        } else {
            const int slices = (int)(word >> 24) == 0 ? 1 : (int)(word >> 24);
            lds = (size_t)CROW_GEMV_ZERO_BYTES + (size_t)waves * (size_t)e->lds_per_wave;
            // a split launch must fit the scratch memory it is given (the kernels check again and report through the status word)
            if (slices > 1 && ((unsigned long long)grid.x * grid.z * (unsigned)slices * (unsigned)(e->nr * e->ns) * 64ull > ws.partial_floats ||
                               (unsigned long long)grid.x * grid.z > ws.counter_slots))
                return CROW_ERR_WORKSPACE;
            geo = (int)(word & 0xFFFFFFu);
            grid.y = (unsigned)slices;
        }
        if (lds > g.lds_cap) return CROW_ERR_SHAPE;
        args[na++] = (void*)&geo;
    }
    if (e->takes_ws) args[na++] = (void*)&ws_arg;
    crow::Geo model_arg = g.model;
    if (e->takes_geo) args[na++] = (void*)&model_arg;
    const bool head = e->stub == (const void*)&gemv_nvfp4_w_argmax;
    // the fused head keeps one key per strip (the kernel checks again and reports through the status word)
    if (head && grid.x > ws.head_words) return CROW_ERR_WORKSPACE;
    hipError_t rc = hipLaunchKernel(stub, grid, block, args, lds, s);
    if (rc == hipSuccess && head) {  // ... and its finishing kernel right behind it: the token out of the strips' keys
        unsigned strips = grid.x;
        void* fargs[3] = {(void*)&vals[6], (void*)&strips, (void*)&ws_arg};
        rc = hipLaunchKernel((const void*)&argmax_finish, dim3(1), dim3(1024), fargs, 0, s);
    }
    if (rc != hipSuccess) (void)hipGetLastError();  // reported here: not left behind for an unrelated later call to find
    return hip_rc(rc);
}

}  // namespace

extern "C" {

int crow_hip_init(int device) {
    if (g.ready) return g.device == device ? CROW_OK : CROW_ERR_BAD_ARGUMENT;
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return (int)e;
    hipDeviceProp_t pr;
    if ((e = hipGetDeviceProperties(&pr, device)) != hipSuccess) return (int)e;
    snprintf(g.name, sizeof g.name, "%s (%s), %d CUs", pr.name, pr.gcnArchName, pr.multiProcessorCount);
    if (strncmp(pr.gcnArchName, "gfx950", 6) != 0) {
        fprintf(stderr, "crow_hip: this library holds gfx950 code objects only; device %d is %s\n", device, pr.gcnArchName);
        return CROW_ERR_BAD_ARGUMENT;
    }
    g.cus = pr.multiProcessorCount;
    g.lds_cap = pr.maxSharedMemoryPerMultiProcessor > 0 ? (size_t)pr.maxSharedMemoryPerMultiProcessor : (size_t)pr.sharedMemPerBlock;
    crow::Workspace ws{};
    ws.partial_floats = PARTIAL_FLOATS;
    ws.counter_slots = COUNTER_SLOTS;
    int* scalars = nullptr;
    // one failure path: everything allocated so far is released again
    auto fail = [&](hipError_t why) {
        (void)hipFree(ws.partials);
        (void)hipFree(ws.counters);
        (void)hipFree(ws.head);
        (void)hipFree(scalars);
        return (int)why;
    };
    if ((e = hipMalloc((void**)&ws.partials, PARTIAL_FLOATS * sizeof(float))) != hipSuccess) return fail(e);
    if ((e = hipMalloc((void**)&ws.counters, COUNTER_WORDS * sizeof(unsigned))) != hipSuccess) return fail(e);
    if ((e = hipMalloc((void**)&ws.head, HEAD_WORDS * sizeof(unsigned long long))) != hipSuccess) return fail(e);
    if ((e = hipMemset(ws.head, 0, HEAD_WORDS * sizeof(unsigned long long))) != hipSuccess) return fail(e);
    ws.head_words = HEAD_WORDS;
    if ((e = hipMalloc((void**)&scalars, 32 * sizeof(int))) != hipSuccess) return fail(e);  // words 0..15: (rows, k_dim) of the layout calls, 16..23: the encoder's maxima, 24: the read probe's sink
    if ((e = hipMemset(ws.counters, 0, COUNTER_WORDS * sizeof(unsigned))) != hipSuccess) return fail(e);
    ws.status = ws.counters + COUNTER_SLOTS;
    if ((e = hipMemcpyToSymbol(HIP_SYMBOL(crow::g_ws), &ws, sizeof ws)) != hipSuccess) return fail(e);
    // a GEMV block of 16 waves, and the GEMM's two staged X tiles, need more dynamic LDS than the default per-block limit
    for (int i = 0; i < g_table_n; i++) {
        size_t most = g_table[i].lds_fixed;
        if (g_table[i].nr != 0) {  // the GEMV family: the largest block the kernel takes, within the device's limit
            most = (size_t)CROW_GEMV_ZERO_BYTES + (size_t)g_table[i].max_waves * (size_t)g_table[i].lds_per_wave;
            if (most > g.lds_cap) most = g.lds_cap;
        }
        if (most > 48 * 1024 &&
            (e = hipFuncSetAttribute(g_table[i].stub, hipFuncAttributeMaxDynamicSharedMemorySize, (int)most)) != hipSuccess)
            return fail(e);
        // the twin for short strips stages up to eight groups of twelve rows per block
        const size_t tile_most = (size_t)CROW_GEMV_ZERO_BYTES + (size_t)CROW_TILE_MAX_GROUPS * (size_t)(g_table[i].lds_per_wave / 2);
        if (g_table[i].tile_stub != nullptr && tile_most > 48 * 1024 &&
            (e = hipFuncSetAttribute(g_table[i].tile_stub, hipFuncAttributeMaxDynamicSharedMemorySize, (int)tile_most)) != hipSuccess)
            return fail(e);
    }
    // `scratch` in host code is a stand-in, not a device address: ask for this device's copy once, and use only that
    unsigned* sp = nullptr;
    if ((e = hipGetSymbolAddress((void**)&sp, HIP_SYMBOL(scratch))) != hipSuccess || sp == nullptr) return fail(e != hipSuccess ? e : hipErrorInvalidSymbol);
    crow::Workspace st{};
    st.partials = (float*)sp;
    st.partial_floats = NOALLOC_PARTIAL_FLOATS;
    st.counters = sp + NOALLOC_PARTIAL_FLOATS;
    st.counter_slots = NOALLOC_COUNTER_SLOTS;
    st.status = st.counters + NOALLOC_COUNTER_SLOTS;
    st.head = (unsigned long long*)(st.status + 32);
    st.head_words = NOALLOC_HEAD_WORDS;
    // counters, status and key start at zero (a process that shut the library down and initialises it again included)
    if ((e = hipMemset(st.counters, 0, (NOALLOC_COUNTER_SLOTS + NOALLOC_TAIL_WORDS) * sizeof(unsigned))) != hipSuccess) return fail(e);
    if ((e = hipDeviceSynchronize()) != hipSuccess) return fail(e);
    g.scalars = scalars;
    g.ws = ws;
    g.ws_static = st;
    g.device = device;
    g.stream = nullptr;
    g.ready = true;
    return CROW_OK;
}

int crow_hip_shutdown(void) {
    if (!g.ready) return CROW_OK;
    (void)hipDeviceSynchronize();
    (void)hipFree(g.ws.partials);
    (void)hipFree(g.ws.counters);
    (void)hipFree(g.ws.head);
    (void)hipFree(g.scalars);
    g = State{};
    return CROW_OK;
}

const char* crow_hip_error_string(int code) {
    switch (code) {
        case CROW_OK: return "ok";
        case CROW_ERR_NOT_INITIALIZED: return "crow_hip_init has not been called";
        case CROW_ERR_KERNEL_MISSING: return "kernel missing";
        case CROW_ERR_BAD_ARGUMENT: return "bad argument";
        case CROW_ERR_ARG_COUNT: return "wrong number of kernel arguments";
        case CROW_ERR_WORKSPACE: return "launch does not fit the split-K workspace";
        case CROW_ERR_SCALE_BYTE: return "scale byte 0xFF in an NVFP4 tensor (no encoder emits it; E4M3 cannot hold 480)";
        case CROW_ERR_SHAPE: return "shape not supported by this kernel";
        case CROW_ERR_GEO: return "geometry not set or out of range (crow_hip_set_geo)";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown crow_hip error";
    }
}

int crow_hip_device_name(char* out, size_t n) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!out || n == 0) return CROW_ERR_BAD_ARGUMENT;
    snprintf(out, n, "%s", g.name);
    return CROW_OK;
}

// The module is the library itself: load/unload exist so that the reference's
// compile -> Module -> get -> unload sequence keeps its shape.
int crow_hip_module_load(crow_module_t* out) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!out) return CROW_ERR_BAD_ARGUMENT;
    *out = (crow_module_t)(void*)g_table;
    return CROW_OK;
}
int crow_hip_module_unload(crow_module_t m) { return m == (crow_module_t)(void*)g_table ? CROW_OK : CROW_ERR_BAD_ARGUMENT; }
int crow_hip_module_get(crow_module_t m, const char* name, crow_fn_t* out) {
    if (m != (crow_module_t)(void*)g_table) return CROW_ERR_BAD_ARGUMENT;
    return crow_hip_get_function(name, out);
}
int crow_hip_get_function(const char* name, crow_fn_t* out) {
    if (!out || !name) return CROW_ERR_BAD_ARGUMENT;
    const FnEntry* e = find(name);
    if (!e) {
        *out = nullptr;
        return CROW_ERR_KERNEL_MISSING;
    }
    *out = (crow_fn_t)(void*)e;
    return CROW_OK;
}
int crow_hip_function_count(void) { return g_table_n; }
const char* crow_hip_function_name(int index) { return index >= 0 && index < g_table_n ? g_table[index].name : nullptr; }
int crow_hip_function_arg_count(crow_fn_t f) {
    const FnEntry* e = entry_of(f);
    return e ? e->nargs : CROW_ERR_BAD_ARGUMENT;
}

int crow_hip_set_geo(int experts, int topk, int hidden, int inter) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (experts < 0 || topk < 0 || hidden < 0 || inter < 0) return CROW_ERR_BAD_ARGUMENT;
    // what the routing kernels take: no routed experts at all, or a power of two of them in 64..1024 with 1..16 picks
    if (experts != 0 && (experts < 64 || experts > 1024 || (experts & (experts - 1)) != 0 || topk < 1 || topk > 16)) return CROW_ERR_GEO;
    // host state only: launches started from now on carry it by value (nothing is copied, nothing waits)
    g.model = crow::Geo{experts, topk, hidden, inter};
    return CROW_OK;
}

int crow_hip_launch(crow_fn_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, const uint64_t* vals, uint32_t n_vals,
                    void* stream) {
    const FnEntry* e = entry_of(f);
    if (!e) return CROW_ERR_KERNEL_MISSING;
    return launch_entry(e, dim3(gx, gy, gz), dim3(bx, 1, 1), vals, n_vals, stream ? (hipStream_t)stream : g.stream, g.ws);
}

int crow_hip_launch_noalloc(crow_fn_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, const uint64_t* vals,
                            uint32_t n_vals, void* stream) {
    const FnEntry* e = entry_of(f);
    if (!e) return CROW_ERR_KERNEL_MISSING;
    // only kernels that are handed their scratch memory as an argument can be pointed at the static array
    if (!e->takes_ws) return CROW_ERR_BAD_ARGUMENT;
    // launch_entry refuses (CROW_ERR_WORKSPACE) a split whose partial sums or counters do not fit what it is given
    return launch_entry(e, dim3(gx, gy, gz), dim3(bx, 1, 1), vals, n_vals, stream ? (hipStream_t)stream : g.stream, g.ws_static);
}

// Which GEMM entry point for m token rows on a [rows, *] tensor.  Up to 16 rows: the K-split body over blocks; up to 96:
// the K-split body with 32-token blocks.  Beyond that the shared-X body, whose blocks are 4 row tiles x MT tokens: the
// dispatcher deals ceil(rows / 256) * ceil(m / MT) blocks over the CUs, so the launch lasts as long as the fullest CU.
// Measured per-block times at K = 5120 (us; they scale with K alike, so only their ratios matter): alone on a CU / sharing it.
const char* crow_hip_gemm_kernel(uint32_t rows, uint32_t m) {
    if (m <= 16) return "gemm_nvfp4_bf16_m16";
    if (m <= 96) return "gemm_nvfp4_bf16_m32";
    // Measured on MI355X at K = 5120 (microseconds): a block of the four-wave kernels alone on a compute unit / each of several
    // sharing one; a block of the eight-wave kernels (one per compute unit: two waves per SIMD) per round of the launch.  The
    // launch lasts as long as the fullest compute unit.
    static const struct { const char* name; uint32_t mt, tiles_per_block; double alone, shared; } cand[] = {
        {"gemm_nvfp4_bf16_m48", 48, 4, 58.0, 45.0},  {"gemm_nvfp4_bf16_m64", 64, 4, 63.0, 48.5},  {"gemm_nvfp4_bf16_m96", 96, 4, 78.0, 78.0},
        {"gemm_nvfp4_bf16_w48", 48, 8, 82.0, 82.0},  {"gemm_nvfp4_bf16_w64", 64, 8, 93.0, 93.0},  {"gemm_nvfp4_bf16_w80", 80, 8, 110.0, 110.0},
        {"gemm_nvfp4_bf16_w96", 96, 8, 118.0, 118.0}};
    const unsigned long long row_tiles = (rows + CROW_TILE_ROWS - 1) / CROW_TILE_ROWS;
    const unsigned long long cus = g.cus > 0 ? (unsigned long long)g.cus : 256ull;
    const char* best = cand[1].name;
    double best_t = 0.0;
    for (const auto& c : cand) {
        const unsigned long long blocks = ((row_tiles + c.tiles_per_block - 1) / c.tiles_per_block) * ((m + c.mt - 1) / c.mt);
        const unsigned long long per_cu = (blocks + cus - 1) / cus;
        const double t = per_cu <= 1 ? c.alone : (double)per_cu * c.shared;
        if (best_t == 0.0 || t < best_t) {
            best_t = t;
            best = c.name;
        }
    }
    return best;
}

// Split of a [rows, k_dim] product over the chip.  A block owns one 16-row strip; the strip's 256-column groups are dealt
// to W waves of the block (combined in LDS) and, only when a strip has more groups than one block's waves can hold, to S
// blocks (combined through the workspace).  The result depends on (rows, k_dim) only.
int crow_hip_launch_dims_split(const char* name, uint32_t rows, uint32_t k_dim, uint32_t z, uint32_t force_s, uint32_t force_w, crow_dims* out) {
    if (!out || !name || rows == 0) return CROW_ERR_BAD_ARGUMENT;
    const FnEntry* e = find(name);
    if (!e) return CROW_ERR_KERNEL_MISSING;
    // CROW_DIMS_COUNT_FROM_MEMORY (verify and token-row kernels only): the launch reads its row count from the word behind
    // m_p / t_p, as the reference's kernels do; the low bits are then the capacity the grid is sized for
    const bool from_memory = (z & CROW_DIMS_COUNT_FROM_MEMORY) != 0 || z == 0;
    z &= ~CROW_DIMS_COUNT_FROM_MEMORY;
    {
        const bool takes_count = strcmp(name, "gemv_nvfp4_wm") == 0 || strcmp(name, "gemv_nvfp4_gum") == 0 || strcmp(name, "gemv_nvfp4_wm_bf16") == 0 ||
                                 strcmp(name, "gemv_nvfp4_gum_bf16") == 0 || strcmp(name, "gemv_fp4_b") == 0 || strcmp(name, "gemv_fp4_b1k") == 0 ||
                                 strcmp(name, "gemv_fp4_bs") == 0;
        if (from_memory && !takes_count) return CROW_ERR_BAD_ARGUMENT;
        if (z == 0) {
            if (strncmp(name, "gemv_nvfp4_", 11) != 0) return CROW_ERR_BAD_ARGUMENT;  // token rows: the capacity sizes the grid
            z = 4;                                                                   // the verify kernels' most
        }
    }
    const uint32_t strips = (rows + CROW_STRIP_ROWS - 1) / CROW_STRIP_ROWS;
    const uint32_t groups = (k_dim + CROW_GROUP_COLS - 1) / CROW_GROUP_COLS;
    const uint32_t rt = (rows + CROW_TILE_ROWS - 1) / CROW_TILE_ROWS, panels = groups;  // the GEMM's 64-row tiles
    if (strcmp(name, "gemv_bf16_w") == 0 || strcmp(name, "gemv_bf16") == 0 || strcmp(name, "gemv_bf16_b") == 0 || strcmp(name, "gemv_b") == 0 ||
        strcmp(name, "gemv_bf16_ws") == 0 || strcmp(name, "gemv_bf16_bs") == 0) {
        // z = T activation rows; whole 16-byte loads: 8 bf16 or 4 f32 weights
        if (k_dim == 0 || k_dim % (strcmp(name, "gemv_b") == 0 ? 4 : 8) != 0) return CROW_ERR_SHAPE;
        if (strcmp(name, "gemv_bf16") == 0 && z != 1) return CROW_ERR_SHAPE;  // the one-token form
        // short tensors: a block of four waves per (row, token); force_w = 4 / 1 asks for one shape or the other
        if (force_w == 4 || (force_w == 0 && (unsigned long long)rows * z <= 2048)) {
            *out = crow_dims{rows, z, 1, 256};
            return CROW_OK;
        }
        *out = crow_dims{(rows + 3) / 4, z, 1, 256};
        return CROW_OK;
    }
    if (e->nr != 0) {  // the NVFP4 GEMV family
        if (k_dim == 0 || k_dim % CROW_BLOCK_VALUES != 0 || k_dim / CROW_BLOCK_VALUES > 0xFFFFFu) return CROW_ERR_SHAPE;
        const uint32_t pairs = k_dim / CROW_BLOCK_VALUES;
        const bool down_combine = strcmp(name, "moe_down_combine") == 0;
        const bool routed = strcmp(name, "gemv_fp4_ptrb") == 0 || strncmp(name, "moe_", 4) == 0;
        const bool tokens = strcmp(name, "gemv_fp4_b") == 0 || strcmp(name, "gemv_fp4_b1k") == 0 || strcmp(name, "gemv_fp4_bs") == 0;
        const bool verify = strcmp(name, "gemv_nvfp4_wm") == 0 || strcmp(name, "gemv_nvfp4_gum") == 0 || strcmp(name, "gemv_nvfp4_wm_bf16") == 0 ||
                            strcmp(name, "gemv_nvfp4_gum_bf16") == 0;
        if (down_combine) {  // rows = hidden; one wave per picked expert, every wave all columns of its strip
            if (g.model.topk < 1 || g.model.topk > 16) return CROW_ERR_GEO;
            *out = crow_dims{strips, pairs | (1u << 24), z, 64u * (uint32_t)g.model.topk};
            return CROW_OK;
        }
        if (e->tile_stub != nullptr && tile_groups(e->nr, pairs) != 0) {
            // about sixteen records per wave; eight waves per block where the staged rows are large (two blocks per compute unit)
            // (force_s / force_w: strips per wave / waves per block, for measurements)
            uint32_t spw = 16u / ((uint32_t)e->nr * groups);
            if (spw < 1) spw = 1;
            if (force_s > 0) spw = force_s > 255 ? 255 : force_s;
            const uint32_t wb = force_w > 0 ? (force_w > 8 ? 8 : force_w) : (groups > 4 ? 8u : 4u), per_block = wb * spw;
            *out = crow_dims{(strips + per_block - 1) / per_block, pairs | (spw << 24), z, 64u * wb};
            return CROW_OK;
        }
        if (verify && z > 4) return CROW_ERR_SHAPE;
        // the fused head keeps one key per strip in the workspace
        if (strcmp(name, "gemv_nvfp4_w_argmax") == 0 && strips > HEAD_WORDS) return CROW_ERR_SHAPE;
        const uint32_t wmax = (uint32_t)e->max_waves / (uint32_t)e->nr;  // waves per tensor in a block
        // A wave walks its run of groups with four of them (9 KB) in flight; few long walks beat many short ones (every wave
        // pays its start, its staging set-up and the block's meeting in LDS once), as long as the launch still has a few
        // thousand waves.  Measured on MI355X: [17408, 5120] one tensor 3 waves per strip (7 groups each), two tensors 2 + 2
        // (10 groups each); [5120, 17408] (68 groups, only 320 strips) 5 slices of 4 waves, which meet through the workspace.
        // A strip stays inside one block up to 64 groups (K = 16384).
        uint32_t w, s;
        if (groups <= 64) {
            const uint32_t per_wave = e->nr == 2 ? 10 : 7;
            w = (groups + per_wave - 1) / per_wave;
            s = 1;
            // (The split depends on the tensor's shape only, never on the number of tokens or experts in the launch: a token's
            // bits are the same in every batch, and the grouped expert kernels reproduce them.  Four waves per tensor at
            // batch 1 would take routed gate|up [1024, 2048] x 8 experts from 8.0 to 7.2 us and give that up.)
        } else {
            w = 4;
            s = (groups + 13) / 14;
        }
        if (force_s > 0) s = force_s;
        if (force_w > 0) w = force_w;
        if (w > wmax) w = wmax;
        if (s > 255) s = 255;
        if (s * w > groups) {  // never more units than groups
            if (w > groups) w = groups;
            s = groups / w;
        }
        const uint32_t gz = routed ? z : (tokens ? (z + 3) / 4 : 1);
        const uint32_t hint = from_memory ? 0 : (verify ? z : (tokens ? (z - 1) % 4 + 1 : 0));
        const uint32_t gx = (strips + (uint32_t)e->ns - 1) / (uint32_t)e->ns;
        *out = crow_dims{gx, pairs | (hint << 20) | (s << 24), gz, 64u * w * (uint32_t)e->nr};
        if (s > 1 && ((unsigned long long)gx * gz * s * (unsigned)(e->nr * e->ns) * 64 > PARTIAL_FLOATS || (unsigned long long)gx * gz > COUNTER_SLOTS)) return CROW_ERR_WORKSPACE;
        return CROW_OK;
    }
    if (strncmp(name, "gemv_nvfp4_w_valu", 17) == 0) {  // a 16-lane group per RG rows, four groups per wave, four waves per block
        if (k_dim == 0 || k_dim % CROW_BLOCK_VALUES != 0) return CROW_ERR_SHAPE;
        const uint32_t per_block = 16u * (uint32_t)(name[17] - '0');
        *out = crow_dims{(rows + per_block - 1) / per_block, 1, 1, 256};
        return CROW_OK;
    }
    if (strncmp(name, "gemm_nvfp4_bf16", 15) == 0) {  // z = M token rows
        if (k_dim == 0 || k_dim % CROW_BLOCK_VALUES != 0) return CROW_ERR_SHAPE;
        if (strcmp(name, "gemm_nvfp4_bf16_m16") == 0) {  // one panel per wave where the workspace allows it
            if (z > 16) return CROW_ERR_SHAPE;
            uint32_t s = (panels + 3) / 4;
            if (s > 16) s = 16;
            while (s > 1 && ((unsigned long long)rt * s * 16 * 64 > PARTIAL_FLOATS || rt > COUNTER_SLOTS)) s--;
            *out = crow_dims{rt, 1, s, 256};
            return CROW_OK;
        }
        if (name[15] == '_' && name[16] == 'w') {  // gemm_nvfp4_bf16_w<tokens per block>: eight row tiles per block
            const uint32_t mtw = (uint32_t)atoi(name + 17);
            *out = crow_dims{(rt + 7) / 8, (z + mtw - 1) / mtw, 1, 512};
            return CROW_OK;
        }
        const uint32_t mt = name[15] == '_' ? (uint32_t)atoi(name + 17) : 128;  // gemm_nvfp4_bf16_m<tokens per block>
        if (mt == 32) {
            *out = crow_dims{rt, (z + 31) / 32, 1, 256};
        } else {
            *out = crow_dims{(rt + 3) / 4, (z + mt - 1) / mt, 1, 256};
        }
        return CROW_OK;
    }
    if (strcmp(name, "repack_nvfp4") == 0 || strcmp(name, "unpack_nvfp4") == 0 || strcmp(name, "dequant_nvfp4_tiled") == 0) {
        *out = crow_dims{groups, strips, 1, 64};
        return CROW_OK;
    }
    if (strcmp(name, "router_top10") == 0) { *out = crow_dims{z, 1, 1, 64}; return CROW_OK; }
    if (strcmp(name, "moe_group") == 0) { *out = crow_dims{1, 1, 1, 1024}; return CROW_OK; }
    if (strcmp(name, "argmax_k") == 0) { *out = crow_dims{1, 1, 1, 1024}; return CROW_OK; }
    if (strcmp(name, "acc_combo") == 0) { *out = crow_dims{(rows + 255) / 256, z, 1, 256}; return CROW_OK; }  // rows = hidden
    if (strcmp(name, "silu_mul_combo") == 0 || strcmp(name, "dequant_fp4_flat") == 0) {  // rows = element count
        *out = crow_dims{(rows + 255) / 256, 1, 1, 256};
        return CROW_OK;
    }
    return CROW_ERR_KERNEL_MISSING;
}

int crow_hip_launch_dims(const char* name, uint32_t rows, uint32_t k_dim, uint32_t z, crow_dims* out) {
    return crow_hip_launch_dims_split(name, rows, k_dim, z, 0, 0, out);
}

int crow_hip_status(void) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    // every stream idle: a launch on another stream (an explicit one, or a graph's) may be in the middle of a hand-over whose
    // arrival counters are cleared below, or may still be about to raise a status bit
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return (int)e;
    unsigned st = 0, st2 = 0;
    if ((e = hipMemcpy(&st, g.ws.status, sizeof st, hipMemcpyDeviceToHost)) != hipSuccess) return (int)e;
    if ((e = hipMemcpy(&st2, g.ws_static.status, sizeof st2, hipMemcpyDeviceToHost)) != hipSuccess) return (int)e;
    if (st == 0 && st2 == 0) return CROW_OK;
    if (st != 0) {
        (void)hipMemset(g.ws.status, 0, sizeof st);
        // a launch that bailed out may have left arrival counters behind
        (void)hipMemset(g.ws.counters, 0, COUNTER_WORDS * sizeof(unsigned));
    }
    if (st2 != 0) (void)hipMemset(g.ws_static.counters, 0, (NOALLOC_COUNTER_SLOTS + NOALLOC_TAIL_WORDS) * sizeof(unsigned));  // counters, status, key
    st |= st2;
    if (st & CROW_STATUS_BAD_SCALE_BYTE) return CROW_ERR_SCALE_BYTE;
    if (st & crow::STATUS_WORKSPACE_TOO_SMALL) return CROW_ERR_WORKSPACE;
    if (st & crow::STATUS_BAD_GEO) return CROW_ERR_GEO;
    return CROW_ERR_SHAPE;
}

int crow_hip_reset_workspace(void) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return (int)e;
    // arrival counters and the status word of both scratch areas (the head's keys need no clearing: every launch overwrites
    // the words it reads)
    if ((e = hipMemset(g.ws_static.counters, 0, (NOALLOC_COUNTER_SLOTS + 32) * sizeof(unsigned))) != hipSuccess) return (int)e;
    return hip_rc(hipMemset(g.ws.counters, 0, COUNTER_WORDS * sizeof(unsigned)));
}

void crow_hip_set_stream(void* stream) { g.stream = (hipStream_t)stream; }
void* crow_hip_cur_stream(void) { return (void*)g.stream; }
int crow_hip_sync(void) { return g.ready ? hip_rc(hipStreamSynchronize(g.stream)) : CROW_ERR_NOT_INITIALIZED; }

int crow_hip_alloc(size_t bytes, void** out) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!out || bytes == 0) return CROW_ERR_BAD_ARGUMENT;
    hipError_t e = hipMalloc(out, bytes);
    if (e != hipSuccess) {
        *out = nullptr;
        return (int)e;
    }
    return hip_rc(hipMemset(*out, 0, bytes));
}
int crow_hip_free(void* p) { return p ? hip_rc(hipFree(p)) : CROW_OK; }
int crow_hip_upload(void* dst, const void* src, size_t bytes) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!dst || !src) return CROW_ERR_BAD_ARGUMENT;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g.stream);
    if (e != hipSuccess) return (int)e;
    return g.stream == nullptr ? hip_rc(hipStreamSynchronize(nullptr)) : CROW_OK;
}
int crow_hip_download(void* dst, const void* src, size_t bytes) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!dst || !src) return CROW_ERR_BAD_ARGUMENT;
    hipError_t e = hipStreamSynchronize(g.stream);
    if (e != hipSuccess) return (int)e;
    return hip_rc(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
}

int crow_hip_event_create(void** out) {
    if (!out) return CROW_ERR_BAD_ARGUMENT;
    hipEvent_t e;
    hipError_t rc = hipEventCreate(&e);
    *out = rc == hipSuccess ? (void*)e : nullptr;
    return hip_rc(rc);
}
int crow_hip_event_record(void* ev) { return ev ? hip_rc(hipEventRecord((hipEvent_t)ev, g.stream)) : CROW_ERR_BAD_ARGUMENT; }
int crow_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
    if (!start || !stop || !ms) return CROW_ERR_BAD_ARGUMENT;
    hipError_t rc = hipEventSynchronize((hipEvent_t)stop);
    if (rc != hipSuccess) return (int)rc;
    return hip_rc(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
}
int crow_hip_event_destroy(void* ev) { return ev ? hip_rc(hipEventDestroy((hipEvent_t)ev)) : CROW_OK; }

int crow_hip_time_launches(crow_fn_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, const uint64_t* vals, uint32_t n_vals,
                           uint32_t n_sets, uint32_t iters, float* us_per_launch) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    const FnEntry* e = entry_of(f);
    if (!e) return CROW_ERR_KERNEL_MISSING;
    if (!vals || !us_per_launch || n_sets == 0 || iters == 0) return CROW_ERR_BAD_ARGUMENT;
    hipEvent_t a, b;
    hipError_t rc;
    if ((rc = hipEventCreate(&a)) != hipSuccess) return (int)rc;
    if ((rc = hipEventCreate(&b)) != hipSuccess) return (int)rc;
    int out = hip_rc(hipEventRecord(a, g.stream));
    for (uint32_t i = 0; i < iters && out == CROW_OK; i++)
        out = launch_entry(e, dim3(gx, gy, gz), dim3(bx), vals + (size_t)(i % n_sets) * n_vals, n_vals, g.stream, g.ws);
    if (out == CROW_OK) out = hip_rc(hipEventRecord(b, g.stream));
    if (out == CROW_OK) out = hip_rc(hipEventSynchronize(b));
    float ms = 0.0f;
    if (out == CROW_OK) out = hip_rc(hipEventElapsedTime(&ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    *us_per_launch = ms * 1000.0f / (float)iters;
    return out;
}

int crow_hip_time_sequence(uint32_t n_kernels, const crow_fn_t* fns, const crow_dims* dims, const uint32_t* n_vals,
                           const uint64_t* vals, uint32_t n_sets, uint32_t iters, float* us_per_iteration) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!fns || !dims || !n_vals || !vals || !us_per_iteration || n_kernels == 0 || n_kernels > 16 || n_sets == 0 || iters == 0)
        return CROW_ERR_BAD_ARGUMENT;
    size_t per_set = 0;
    for (uint32_t k = 0; k < n_kernels; k++) {
        if (!entry_of(fns[k])) return CROW_ERR_KERNEL_MISSING;
        per_set += n_vals[k];
    }
    hipEvent_t a, b;
    hipError_t rc;
    if ((rc = hipEventCreate(&a)) != hipSuccess) return (int)rc;
    if ((rc = hipEventCreate(&b)) != hipSuccess) return (int)rc;
    int out = hip_rc(hipEventRecord(a, g.stream));
    for (uint32_t i = 0; i < iters && out == CROW_OK; i++) {
        const uint64_t* v = vals + (size_t)(i % n_sets) * per_set;
        for (uint32_t k = 0; k < n_kernels && out == CROW_OK; k++) {
            out = launch_entry((const FnEntry*)(void*)fns[k], dim3(dims[k].gx, dims[k].gy, dims[k].gz), dim3(dims[k].bx), v, n_vals[k], g.stream, g.ws);
            v += n_vals[k];
        }
    }
    if (out == CROW_OK) out = hip_rc(hipEventRecord(b, g.stream));
    if (out == CROW_OK) out = hip_rc(hipEventSynchronize(b));
    float ms = 0.0f;
    if (out == CROW_OK) out = hip_rc(hipEventElapsedTime(&ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    *us_per_iteration = ms * 1000.0f / (float)iters;
    return out;
}

int crow_hip_time_pure_read(const uint64_t* bufs, uint32_t n_bufs, size_t bytes, uint32_t blocks, uint32_t threads, uint32_t pattern, uint32_t iters, float* us_per_launch) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!bufs || !us_per_launch || n_bufs == 0 || iters == 0 || blocks == 0 || threads == 0 || threads % 64 != 0 || threads > 1024 || pattern > 2) return CROW_ERR_BAD_ARGUMENT;
    if (bytes == 0 || bytes % CROW_GROUP_BYTES != 0 || bytes / CROW_GROUP_BYTES > 0xFFFFFFFFull) return CROW_ERR_SHAPE;
    unsigned units = (unsigned)(bytes / CROW_GROUP_BYTES);
    unsigned* sink = (unsigned*)(g.scalars + 24);
    hipEvent_t a, b;
    hipError_t rc;
    if ((rc = hipEventCreate(&a)) != hipSuccess) return (int)rc;
    if ((rc = hipEventCreate(&b)) != hipSuccess) return (int)rc;
    int out = hip_rc(hipEventRecord(a, g.stream));
    for (uint32_t i = 0; i < iters && out == CROW_OK; i++) {
        const unsigned char* w = (const unsigned char*)(uintptr_t)bufs[i % n_bufs];
        if (pattern == 0) {
            void* args[3] = {(void*)&w, (void*)&units, (void*)&sink};
            out = hip_rc(hipLaunchKernel((const void*)&pure_read_groups, dim3(blocks), dim3(threads), args, 0, g.stream));
        } else {
            size_t n16 = bytes / 16;
            void* args[3] = {(void*)&w, (void*)&n16, (void*)&sink};
            out = hip_rc(hipLaunchKernel(pattern == 1 ? (const void*)&pure_read_flat_nt : (const void*)&pure_read_flat, dim3(blocks), dim3(threads), args, 0, g.stream));
        }
    }
    if (out == CROW_OK) out = hip_rc(hipEventRecord(b, g.stream));
    if (out == CROW_OK) out = hip_rc(hipEventSynchronize(b));
    float ms = 0.0f;
    if (out == CROW_OK) out = hip_rc(hipEventElapsedTime(&ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    *us_per_launch = ms * 1000.0f / (float)iters;
    return out;
}

int crow_hip_stream_create(void** out) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!out) return CROW_ERR_BAD_ARGUMENT;
    hipStream_t s = nullptr;
    const int rc = hip_rc(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *out = (void*)s;
    return rc;
}
int crow_hip_stream_destroy(void* stream) {
    if (!stream) return CROW_OK;
    if (g.stream == (hipStream_t)stream) g.stream = nullptr;
    return hip_rc(hipStreamDestroy((hipStream_t)stream));
}
int crow_hip_begin_capture(void* stream) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!stream) return CROW_ERR_BAD_ARGUMENT;  // the legacy default stream cannot be captured
    g.stream = (hipStream_t)stream;
    return hip_rc(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeGlobal));
}
int crow_hip_end_capture_instantiate(void* stream, void** graph_exec_out) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!stream || !graph_exec_out) return CROW_ERR_BAD_ARGUMENT;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture((hipStream_t)stream, &graph);
    if (e != hipSuccess) return (int)e;
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);  // the executable graph is independent of its template
    if (e != hipSuccess) return (int)e;
    *graph_exec_out = (void*)exec;
    return CROW_OK;
}
int crow_hip_launch_graph(void* graph_exec, void* stream) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!graph_exec) return CROW_ERR_BAD_ARGUMENT;
    return hip_rc(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
}
int crow_hip_graph_exec_destroy(void* graph_exec) {
    if (!graph_exec) return CROW_OK;
    return hip_rc(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
}
int crow_hip_time_graph(void* graph_exec, void* stream, uint32_t iters, float* us_per_replay) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!graph_exec || !us_per_replay || iters == 0) return CROW_ERR_BAD_ARGUMENT;
    hipEvent_t a, b;
    hipError_t rc;
    if ((rc = hipEventCreate(&a)) != hipSuccess) return (int)rc;
    if ((rc = hipEventCreate(&b)) != hipSuccess) return (int)rc;
    int out = hip_rc(hipEventRecord(a, (hipStream_t)stream));
    for (uint32_t i = 0; i < iters && out == CROW_OK; i++) out = hip_rc(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
    if (out == CROW_OK) out = hip_rc(hipEventRecord(b, (hipStream_t)stream));
    if (out == CROW_OK) out = hip_rc(hipEventSynchronize(b));
    float ms = 0.0f;
    if (out == CROW_OK) out = hip_rc(hipEventElapsedTime(&ms, a, b));
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    *us_per_replay = ms * 1000.0f / (float)iters;
    return out;
}

#ifdef CROW_TRACE  // measurement builds only: the per-block timestamps of gemv.h
int crow_hip_trace_read(unsigned long long* dst, size_t words, int clear) {
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return (int)e;
    if ((e = hipMemcpyFromSymbol(dst, HIP_SYMBOL(crow::crow_trace), words * 8)) != hipSuccess) return (int)e;
    if (clear) {
        void* p = nullptr;
        if ((e = hipGetSymbolAddress(&p, HIP_SYMBOL(crow::crow_trace))) != hipSuccess) return (int)e;
        return hip_rc(hipMemset(p, 0, sizeof(unsigned long long) * 16384 * 8));
    }
    return CROW_OK;
}
#endif

size_t crow_hip_container_bytes(uint32_t rows, uint32_t cols) { return crow_container_bytes(rows, cols); }
size_t crow_hip_tiled_bytes(uint32_t rows, uint32_t cols) { return crow_tiled_bytes(rows, cols); }
uint32_t crow_hip_tile_code_offset(uint32_t row, uint32_t wp) { return row < 16 && wp < 32 ? crow_group_code_offset(row, wp) : UINT32_MAX; }
uint32_t crow_hip_tile_scale_offset(uint32_t row, uint32_t sb) { return row < 16 && sb < 16 ? crow_group_scale_offset(row, sb) : UINT32_MAX; }

static int layout_launch(const char* name, const void* a, const void* b, const void* c, uint32_t rows, uint32_t cols) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!a || !b || rows == 0 || cols == 0 || cols % CROW_BLOCK_VALUES != 0) return a && b ? CROW_ERR_SHAPE : CROW_ERR_BAD_ARGUMENT;
    // the two scalars ride in a small ring of device words so that back-to-back calls do not race
    static int slot = 0;
    int* sc = g.scalars + 2 * (slot++ & 7);
    int host[2] = {(int)rows, (int)cols};
    hipError_t e = hipMemcpyAsync(sc, host, sizeof host, hipMemcpyHostToDevice, g.stream);
    if (e != hipSuccess) return (int)e;
    if ((e = hipStreamSynchronize(g.stream)) != hipSuccess) return (int)e;  // `host` is a stack buffer
    crow_dims d;
    int rc = crow_hip_launch_dims(name, rows, cols, 1, &d);
    if (rc != CROW_OK) return rc;
    uint64_t vals[5];
    uint32_t n = 0;
    vals[n++] = (uint64_t)a;
    vals[n++] = (uint64_t)b;
    if (c) vals[n++] = (uint64_t)c;
    vals[n++] = (uint64_t)sc;
    vals[n++] = (uint64_t)(sc + 1);
    rc = launch_entry(find(name), dim3(d.gx, d.gy, d.gz), dim3(d.bx), vals, n, g.stream, g.ws);
    if (rc != CROW_OK) return rc;
    return crow_hip_status();
}

int crow_hip_quantize_nvfp4(const float* values_dev, size_t n_values, void* blocks_dev, float* global_scale_dev) {
    if (!g.ready) return CROW_ERR_NOT_INITIALIZED;
    if (!values_dev || !blocks_dev || !global_scale_dev) return CROW_ERR_BAD_ARGUMENT;
    if (n_values == 0 || n_values % CROW_BLOCK_VALUES != 0) return CROW_ERR_SHAPE;
    // the tensor's largest raw scale meets in one device word (one of the library's own, taken in turn so that calls in a
    // row do not share it)
    static std::atomic<unsigned> slot{0};
    unsigned* max_bits = (unsigned*)(g.scalars + 16 + (slot.fetch_add(1) & 7u));
    hipError_t e;
    void* a0[1] = {(void*)&max_bits};
    if ((e = hipLaunchKernel((const void*)&quantize_nvfp4_clear, dim3(1), dim3(1), a0, 0, g.stream)) != hipSuccess) return (int)e;
    unsigned long long n_sub = n_values / 16;
    const unsigned long long want = (n_sub + 255) / 256;
    const unsigned blocks1 = (unsigned)(want < 2048 ? want : 2048);
    const float* vals = values_dev;
    unsigned char* out = (unsigned char*)blocks_dev;
    const unsigned* max_ro = max_bits;
    void* a1[3] = {(void*)&vals, (void*)&n_sub, (void*)&max_bits};
    if ((e = hipLaunchKernel((const void*)&quantize_nvfp4_amax, dim3(blocks1), dim3(256), a1, 0, g.stream)) != hipSuccess) return (int)e;
    if (want > 0x7FFFFFFFull) return CROW_ERR_SHAPE;
    void* a2[5] = {(void*)&vals, (void*)&n_sub, (void*)&max_ro, (void*)&out, (void*)&global_scale_dev};
    return hip_rc(hipLaunchKernel((const void*)&quantize_nvfp4_encode, dim3((unsigned)want), dim3(256), a2, 0, g.stream));
}

int crow_hip_repack_nvfp4(const void* src_dev, uint32_t rows, uint32_t cols, void* dst_dev) {
    return layout_launch("repack_nvfp4", src_dev, dst_dev, nullptr, rows, cols);
}
int crow_hip_unpack_nvfp4(const void* src_dev, uint32_t rows, uint32_t cols, void* dst_dev) {
    return layout_launch("unpack_nvfp4", src_dev, dst_dev, nullptr, rows, cols);
}
int crow_hip_dequant_tiled(const void* w_dev, const float* gs_dev, uint32_t rows, uint32_t cols, float* out_dev) {
    return layout_launch("dequant_nvfp4_tiled", w_dev, gs_dev, out_dev, rows, cols);
}

}  // extern "C"

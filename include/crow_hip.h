/*
 * libcrow_hip.so - the C ABI of the MI355X (gfx950) NVFP4 weight x activation library.
 *
 * It replaces, for the NVFP4 hot path only, the reference engine's NVRTC compile/launch layer:
 *   engine/src/cuda.rs:274-284      compile(src) -> Module            -> crow_hip_module_load
 *   engine/src/cuda.rs:485-509      Module::get(name), Module::unload -> crow_hip_module_get / _unload
 *   engine/src/kernels.rs:5128-5240 Kernels::new / Kernels::f(name)   -> crow_hip_get_function
 *   engine/src/kernels.rs:5284-5348 launch_v / launch_sync            -> crow_hip_launch (+ crow_hip_sync)
 *   engine/src/kernels.rs:5040-5125 KernelGeo prelude (CN_* defines)  -> crow_hip_set_geo
 *   engine/src/cuda.rs:398-687      alloc / free / upload / dtoh      -> crow_hip_alloc ... crow_hip_download
 *   engine/src/cuda.rs:13-24        set_stream / cur_stream           -> crow_hip_set_stream / crow_hip_cur_stream
 *   engine/src/weights.rs:26-33, gen.rs:2178-2198 (load_fp4 + the 0x7F rule) -> crow_hip_repack_nvfp4
 * The code objects are built ahead of time for gfx950 and live inside the library; nothing is
 * compiled at run time.  Plain pointers and sizes only; every call returns 0 on success or a
 * negative crow_status / a positive hipError_t, never aborts and never throws.
 *
 * Kernel arguments keep the reference convention: every value handed to crow_hip_launch is a
 * 64-bit device address; scalars live in 4-byte device words.  Weight pointers are to tensors in
 * the library's tiled layout (crow_hip_repack_nvfp4), not to raw container bytes.
 * crow_kernels.h lists every kernel name with its value list and the reference kernel it stands for.
 *
 * Threading: like the reference engine (one engine thread, one process-global current stream)
 * the library keeps one workspace per process; launches that use it must be ordered on one stream.
 */
#ifndef CROW_HIP_H
#define CROW_HIP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct crow_fn_s* crow_fn_t;     /* opaque kernel handle (CUfunction in the reference) */
typedef struct crow_module_s* crow_module_t; /* opaque module handle (CUmodule in the reference) */

enum crow_status {
    CROW_OK = 0,
    CROW_ERR_NOT_INITIALIZED = -1,
    CROW_ERR_KERNEL_MISSING = -2, /* the Rust shim turns this into panic!("kernel missing: {name}") */
    CROW_ERR_BAD_ARGUMENT = -3,
    CROW_ERR_ARG_COUNT = -4,      /* launch with a different number of values than the kernel takes */
    CROW_ERR_WORKSPACE = -5,      /* a launch needed more split-K workspace than the library holds */
    CROW_ERR_SCALE_BYTE = -6,     /* repack met scale byte 0xFF (reads 480 in the reference; E4M3 cannot hold it) */
    CROW_ERR_SHAPE = -7,
    CROW_ERR_GEO = -8
};

/* launch geometry chosen by the library for a kernel and a problem (wave64 shapes stay out of the caller).  The four words
 * are to be handed to crow_hip_launch unchanged.  For the NVFP4 GEMV family `gy` is not a grid extent: it carries the problem
 * (bits 0..19 = k_dim / 64, bits 20..23 = activation rows of the last token group or 0, bits 24..31 = column slices per
 * strip); crow_hip_launch launches (gx, slices, gz) blocks and hands the low 24 bits to the kernel by value, so that a wave
 * can address its weights before the words behind k_dim_p / m_p have arrived from memory. */
typedef struct crow_dims {
    uint32_t gx, gy, gz, bx;
} crow_dims;

/* ---- lifetime ---- */
int crow_hip_init(int device);            /* Ctx::init, engine/src/cuda.rs:435 */
int crow_hip_shutdown(void);
const char* crow_hip_error_string(int code);
int crow_hip_device_name(char* out, size_t n);

/* ---- module / kernel table ---- */
int crow_hip_module_load(crow_module_t* out);
int crow_hip_module_unload(crow_module_t m);
int crow_hip_module_get(crow_module_t m, const char* name, crow_fn_t* out);
int crow_hip_get_function(const char* name, crow_fn_t* out);
int crow_hip_function_count(void);
const char* crow_hip_function_name(int index);
int crow_hip_function_arg_count(crow_fn_t f);

/* ---- geometry the reference compiles into its kernel text ----
 * Host state only: the launcher hands it BY VALUE to the kernels that need it (router_top10, moe_route_gate_up_silu,
 * moe_down_combine, moe_group, silu_mul_combo, acc_combo), so the call copies nothing to the device and waits for nothing,
 * launches already queued keep the geometry they were started with, and a launch captured into a graph keeps the
 * geometry it was captured with.  A process that serves two geometries sets the one it needs before each group of launches. */
int crow_hip_set_geo(int experts, int topk, int hidden, int inter);

/* ---- launch ---- */
int crow_hip_launch(crow_fn_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, const uint64_t* vals,
                    uint32_t n_vals, void* stream);
/* crow_hip_launch for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and results as crow_hip_launch,
 * for the kernels that use scratch memory (the NVFP4 GEMV family; any other kernel: CROW_ERR_BAD_ARGUMENT),
 * but their scratch - split-K partial sums, arrival counters, the status word, the fused head's keys - is a fixed array
 * inside the library's code object (CROW_NOALLOC_SCRATCH_BYTES per device, held until the process ends) instead of the
 * workspace crow_hip_init allocates; the call itself allocates and frees nothing.  A split launch (column slices S > 1 in
 * `gy`) with more than CROW_NOALLOC_MAX_PARTIAL_FLOATS partial sums (gx * gz * S * tensors * 64) or more than
 * CROW_NOALLOC_MAX_STRIPS strips (gx * gz), and a fused head (gemv_nvfp4_w_argmax) of more than CROW_NOALLOC_MAX_HEAD_STRIPS
 * strips, is refused with CROW_ERR_WORKSPACE before anything runs.  Every call on a device
 * shares the one array: calls that overlap on the device (two streams, two threads) race; order them on one stream.  (The
 * library cannot check this for the caller: telling whether an earlier launch on another stream is still running takes a
 * stream query, which is not legal while a stream is being captured in global mode - the very callers this entry point
 * is for.)  crow_hip_status reports both scratch areas; crow_hip_reset_workspace clears the counters and status words of both. */
#define CROW_NOALLOC_MAX_PARTIAL_FLOATS (1u << 20)
#define CROW_NOALLOC_MAX_STRIPS 4096u
#define CROW_NOALLOC_MAX_HEAD_STRIPS 16384u /* the fused head through this entry point: at most 262,144 rows */
#define CROW_NOALLOC_SCRATCH_BYTES (4u * (CROW_NOALLOC_MAX_PARTIAL_FLOATS + CROW_NOALLOC_MAX_STRIPS + 32u + 2u * CROW_NOALLOC_MAX_HEAD_STRIPS))
int crow_hip_launch_noalloc(crow_fn_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, const uint64_t* vals,
                            uint32_t n_vals, void* stream);
/* grid/block for `name` on a [rows, k_dim] tensor with `z` token rows (batched and verify kernels: the value *t_p / *m_p
 * will hold) or combos (routed kernels); 1 otherwise.  The split of the work depends on (rows, k_dim) only, never on z.
 *
 * Dimensions made for a row count are BOUND to it: the count rides in `gy`, the kernel works with it from its first
 * instruction and stores nothing (CROW_ERR_SHAPE from crow_hip_status) if the word behind m_p / t_p says otherwise - so a
 * launch captured into a graph with such dimensions serves that one count.  For the reference's own convention - a fixed
 * grid, the count read from the device word by every launch (engine/src/kernels_p2.rs:472-497, gen.rs:5455-5466 rewrite
 * *m_p per step) - pass z = CROW_DIMS_COUNT_FROM_MEMORY | capacity: the verify kernels (gemv_nvfp4_wm / _gum and their
 * bf16 twins; capacity 1..4, or plain z = 0) then serve any 1 <= *m_p <= 4 with one set of dimensions and one captured
 * graph, the token-row kernels (gemv_fp4_b / _b1k / _bs) any 1 <= *t_p <= capacity.  Row m of such a launch holds the same
 * bits as under dimensions bound to the count; the only cost is one dependent read before the first weight request.
 *
 * Precondition of every launch of the NVFP4 GEMV family: the four words come from this call for the SAME (rows, k_dim) as
 * the weight tensor handed to the kernel.  The kernels read their weights as the dimensions say before they compare K and
 * the row count with the caller's device words (a disagreement stores nothing and raises CROW_ERR_SHAPE) - dimensions
 * made for a larger tensor make them read beyond the allocation. */
#define CROW_DIMS_COUNT_FROM_MEMORY 0x80000000u
int crow_hip_launch_dims(const char* name, uint32_t rows, uint32_t k_dim, uint32_t z, crow_dims* out);
/* the GEMM entry point (a name of the kernel table) that serves `m` token rows fastest on a tensor of `rows` rows: the
 * choice depends on how the blocks of each tiling fall on this device's compute units */
const char* crow_hip_gemm_kernel(uint32_t rows, uint32_t m);
/* reads and clears the device status word (waits for the whole device first: every stream): CROW_OK or CROW_ERR_* */
int crow_hip_status(void);
int crow_hip_reset_workspace(void);

/* ---- streams and memory (thin shims over HIP) ---- */
void crow_hip_set_stream(void* stream);
void* crow_hip_cur_stream(void);
int crow_hip_sync(void);
int crow_hip_alloc(size_t bytes, void** out);   /* zero-filled, like alloc_named (engine/src/cuda.rs:398-427) */
int crow_hip_free(void* p);
int crow_hip_upload(void* dst, const void* src, size_t bytes);   /* upload_into: async on a capture stream, else + sync */
int crow_hip_download(void* dst, const void* src, size_t bytes); /* dtoh: blocking */

/* ---- timing on the current stream (HIP events; what CROW_KPROF books per launch in the reference,
 * engine/src/kernels.rs:5245-5280, is measured by the caller with these) ---- */
int crow_hip_event_create(void** out);
int crow_hip_event_record(void* ev);                              /* on the current stream */
int crow_hip_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for `stop` */
int crow_hip_event_destroy(void* ev);

/* ---- graph capture: cuda::stream_create_non_blocking / begin_capture / end_capture_instantiate / launch_graph /
 * graph_exec_destroy / stream_destroy, engine/src/cuda.rs:113-203.  A launch sequence issued with crow_hip_launch
 * between begin and end on a created stream is recorded, not run (no host read, no synchronisation, no allocation and
 * no memset happens inside crow_hip_launch); the instantiated graph replays it.  Capture mode is global, as the
 * reference's.  Default stream priority only. ---- */
int crow_hip_stream_create(void** out);         /* non-blocking stream */
int crow_hip_stream_destroy(void* stream);
int crow_hip_begin_capture(void* stream);       /* also makes `stream` the current stream, as the reference's capture path does */
int crow_hip_end_capture_instantiate(void* stream, void** graph_exec_out); /* the template graph is destroyed */
int crow_hip_launch_graph(void* graph_exec, void* stream);
int crow_hip_graph_exec_destroy(void* graph_exec);

/* ---- load-time repack (the one call the reference does not have) ---- */
size_t crow_hip_container_bytes(uint32_t rows, uint32_t cols);
size_t crow_hip_tiled_bytes(uint32_t rows, uint32_t cols);
/* where the repacker puts things inside a 2304-byte group of 16 rows x 256 columns (host arithmetic, no device needed): the
 * byte offset of the code dword of strip row `row` (0..15), group columns 8 wp .. 8 wp + 7 (wp 0..31), and of the scale byte
 * of strip row `row`, 16-column sub-block sb (0..15).  Group (strip, gi) of a tensor starts at
 * (strip * ceil(cols / 256) + gi) * 2304.  UINT32_MAX for an argument out of range. */
uint32_t crow_hip_tile_code_offset(uint32_t row, uint32_t wp);
uint32_t crow_hip_tile_scale_offset(uint32_t row, uint32_t sb);
/* ---- the NVFP4 encoder, ceiling scales: quantize_nvfp4 with ScalesMode::Ceil of converter/src/main.rs:550-664
 * (encode_ue4m3_ceil :141-169, encode_subblock_ceil :404-410, e2m1_index :111-119), on the device.
 * values_dev: n_values f32 (a multiple of 64; sub-blocks are 16 consecutive values); blocks_dev: n_values / 64 * 36 bytes of
 * container blocks (4 scale bytes + 32 code bytes each); *global_scale_dev: max(amax / 6) / 448, or 1 for an all-zero
 * tensor.  Byte for byte what the converter writes (every `/` of its arithmetic a correctly rounded division, the codes
 * chosen against the reciprocal of the decoded scale), so the result loads through crow_hip_repack_nvfp4 like any
 * container tensor.  Asynchronous on the current stream. ---- */
int crow_hip_quantize_nvfp4(const float* values_dev, size_t n_values, void* blocks_dev, float* global_scale_dev);

/* src_dev: container bytes [rows][cols/64][36] already on the device; dst_dev: crow_hip_tiled_bytes.
 * Applies the scale rule (0x7F -> 0x7E).  Expert tensors [E][rows][cols]: call once per expert
 * slab, the tiled slabs are then contiguous per expert. */
int crow_hip_repack_nvfp4(const void* src_dev, uint32_t rows, uint32_t cols, void* dst_dev);
int crow_hip_unpack_nvfp4(const void* src_dev, uint32_t rows, uint32_t cols, void* dst_dev);
/* out_dev: f32 [rows][cols], bit-exact with the reference decode after the scale rule */
int crow_hip_dequant_tiled(const void* w_dev, const float* gs_dev, uint32_t rows, uint32_t cols, float* out_dev);

#ifdef __cplusplus
}
#endif
#endif

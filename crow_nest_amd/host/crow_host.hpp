// Host side of the NVFP4 path in C++, above the C ABI of include/crow_hip.h: the types and functions a maintainer of
// the reference engine (Rust) finds under the same names with the same argument meaning and the same failure
// behaviour.  Where the reference panics, these throw crow::Panic carrying the panic's text; where it returns
// Err(String), they throw crow::Refused carrying that string.
//
//   reference                                            here
//   cuda::Ctx::init                 cuda.rs:435          crow::Ctx::init
//   cuda::compile / Module          cuda.rs:274-284,485  crow::compile / crow::Module {get, unload}
//   Kernels::new / f                kernels.rs:5128-5240 crow::Kernels {f}: "kernel missing: {name}"
//   launch_v / launch_sync          kernels.rs:5284-5348 crow::launch_v / launch_sync
//   cuda::alloc_named, upload_into, dtoh, sync           crow::DevBuf {upload, download}, crow::sync
//   Params (device scalar words)    gen.rs:2913-2925     crow::Params {i32}
//   cpu_nvfp4::Nvfp4Matrix          cpu_nvfp4.rs:107-141 crow::Nvfp4Matrix
//   weights::load_fp4, PW::Fp4      weights.rs:26-33, gen.rs:234-237   crow::load_fp4, crow::Fp4 {w, gs}
//   dense_proj / dense_ffn_w / proj_m / lm_head_row / moe_run           crow::Engine (gen.rs:3915-3992, 5455-5466,
//                                                        4766-4784, 4168-4534)
//   Cnq::open_checked / find / byte_len / read_bytes / read_range       crow::Cnq (cnq.rs:143-239, 715-733, 952-1135)
// Nothing here computes on the CPU: without the HIP library and a gfx950 device every entry fails loudly.
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/crow_hip.h"

namespace crow {

struct Panic : std::runtime_error {
    using std::runtime_error::runtime_error;
};
struct Refused : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// cuda::ck (cuda.rs:286-313): a failing call is fatal, with the call's name and the error's text
void ck(int rc, const char* what);

struct Ctx {
    static void init(int device = 0);  // cuda.rs:435: device, workspace, kernel table
    static bool ready();
};
void sync();    // cuda::sync, cuda.rs:716
void status();  // throws Panic if a launch since the last call refused its shape or did not fit the workspace

// a device allocation owned by the host side (alloc_named / free_dev with Drop)
class DevBuf {
  public:
    DevBuf() = default;
    explicit DevBuf(size_t bytes);
    DevBuf(DevBuf&& o) noexcept : p_(o.p_), n_(o.n_) { o.p_ = nullptr, o.n_ = 0; }
    DevBuf& operator=(DevBuf&& o) noexcept;
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    ~DevBuf();
    uint64_t ptr() const { return (uint64_t)(uintptr_t)p_; }
    size_t bytes() const { return n_; }
    void upload(const void* src, size_t bytes, size_t at = 0);         // upload_into, cuda.rs:625
    void download(void* dst, size_t bytes, size_t at = 0) const;       // dtoh, cuda.rs:664 (synchronises the stream)

  private:
    void* p_ = nullptr;
    size_t n_ = 0;
};

// the geometry the reference bakes into its kernel source (kernels.rs:5040-5125, CN_* defines)
struct KernelGeo {
    int experts = 0, topk = 0, hidden = 0, inter = 0;
};

class Module {
  public:
    explicit Module(crow_module_t h) : h_(h) {}
    crow_fn_t get(const char* name) const;  // Module::get, cuda.rs:500: Panic "kernel missing: {name}"
    void unload();                          // cuda.rs:490
  private:
    crow_module_t h_;
};
Module compile(const KernelGeo* geo = nullptr);  // cuda::compile, cuda.rs:274: loads the ahead-of-time objects, writes the geometry
void set_geo(const KernelGeo& geo);

class Kernels {
  public:
    explicit Kernels(const Module& m);          // Kernels::new: every launched name resolved once
    crow_fn_t f(const std::string& name) const; // Panic "kernel missing: {name}" (kernels.rs:5238)
  private:
    std::map<std::string, crow_fn_t> map_;
};

struct Dims {
    uint32_t gx, gy, gz, bx;
};
Dims launch_dims(const char* name, uint32_t rows, uint32_t k_dim, uint32_t z = 1);
void launch_v(crow_fn_t f, const Dims& d, const std::vector<uint64_t>& vals);  // asynchronous, current stream
void launch_v(crow_fn_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, const std::vector<uint64_t>& vals);
void launch_sync(crow_fn_t f, const Dims& d, const std::vector<uint64_t>& vals);

// device words for kernel scalars, created on demand
class Params {
  public:
    uint64_t i32(int v);
  private:
    std::map<int, DevBuf> words_;
};

// one NVFP4 matrix [rows, cols] over container bytes on the host (borrowed)
struct Nvfp4Matrix {
    const uint8_t* bytes;
    size_t len;
    int rows, cols;
    float global_scale;
    static size_t byte_len(int rows, int cols) { return (size_t)rows * (size_t)(cols / 64) * 36; }
    // Refused "cpu_nvfp4: {cols} columns are not whole 64-value NVFP4 blocks" / "cpu_nvfp4: [{rows}, {cols}] needs {n} B, got {m}"
    static Nvfp4Matrix make(const uint8_t* bytes, size_t len, int rows, int cols, float global_scale);
};

// one routed expert on the host (cpu_nvfp4::ExpertBlock, cpu_nvfp4.rs:143-179): gate [inter, hidden], up [inter, hidden],
// down [hidden, inter].  Refused "cpu_nvfp4: expert shapes gate [..], up [..], down [..] do not fit together" /
// "cpu_nvfp4: expert unit H {hidden} I {inter} needs {n} B, got {m}"
struct ExpertBlock {
    Nvfp4Matrix gate, up, down;
    int hidden, inter;
    static ExpertBlock make(const Nvfp4Matrix& gate, const Nvfp4Matrix& up, const Nvfp4Matrix& down);
    // one expert unit as the GLM converter writes it: gate | up | down back to back, global scales in that order
    static ExpertBlock from_unit(const uint8_t* unit, size_t len, int hidden, int inter, const float (&global_scales)[3]);
};

// PW::Fp4(w, gs): tiled weight bytes and the global scale, both on the device
struct Fp4 {
    DevBuf w, gs;
    int rows = 0, cols = 0;
};
Fp4 load_fp4(const Nvfp4Matrix& m);  // upload, re-tile on the device (the 0x7F -> 0x7E scale rule is applied there)
std::vector<float> dequant(const Fp4& w);  // f32 [rows][cols], bit-exact with the reference decode after the scale rule

// quantize_nvfp4(values, Ceil) of the converter (converter/src/main.rs:534-664) on the device: container blocks (36 bytes per 64
// values) and the tensor's global scale, byte for byte what the converter writes.  Panics, as the converter's assert does, when
// the value count is not whole 64-value blocks.
struct QuantizedNvfp4 {
    std::vector<uint8_t> blocks;
    float global_scale = 1.0f;
};
QuantizedNvfp4 quantize_nvfp4(const float* values, size_t n_values);

struct MlpW {
    Fp4 gate, up, down;
};
MlpW load_expert_block(const ExpertBlock& e);  // the unit's three matrices on the device, each under its own global scale

// an expert tensor [E][rows][cols] re-tiled per expert: slab e starts at e * slab_bytes (residency.rs:108-117)
struct ExpertSlabs {
    DevBuf w, gs;
    int experts = 0, rows = 0, cols = 0;
    size_t slab_bytes = 0;
    uint64_t ptr(int e) const { return w.ptr() + (uint64_t)e * slab_bytes; }
};
ExpertSlabs load_expert_slabs(const uint8_t* data, size_t len, int experts, int rows, int cols, float global_scale);
struct MoeW {
    ExpertSlabs gate_up;  // [E][2 I][H], gate rows 0..I, up rows I..2I
    ExpertSlabs down;     // [E][H][I]
    DevBuf table;         // u64 [E][2]: device address of expert e's gate_up / down slab
};
MoeW make_moe(ExpertSlabs gate_up, ExpertSlabs down);

constexpr int NVFP4_MMAX = 4;  // kernels_p2.rs:397

// The callers of the hot path (engine/src/gen.rs).  x, h, y, logits are device addresses of f32 buffers the caller owns
// (x may be bf16 where `x_bf16` says so); every launch goes through launch_v(k.f(name), ...).
class Engine {
  public:
    explicit Engine(const KernelGeo* geo = nullptr);
    // gen.rs:3915-3932: t == 1 -> gemv_nvfp4_w; 2..4 -> gemv_nvfp4_wm; more -> GEMM (bf16 x) or gemv_fp4_b (f32 x)
    void dense_proj(const Fp4& w, int t, uint64_t x, uint64_t y, bool x_bf16 = false);
    // gen.rs:5455-5466: gemv_nvfp4_wm over M <= 4 rows; Panic outside 1..=4
    void proj_m(const Fp4& w, int m, uint64_t x, uint64_t y, bool x_bf16 = false);
    // h[t][I] = silu(gate x) * up x in one launch (t <= 4)
    void gate_up(const MlpW& mlp, int t, uint64_t x, uint64_t h, bool x_bf16 = false);
    // gen.rs:3974-3992: down(silu(gate x) * up x) over t <= 4 rows; h is scratch [t][I]
    void dense_ffn_w(const MlpW& mlp, uint64_t x, int t, uint64_t h, uint64_t y, bool x_bf16 = false);
    // gen.rs:4766-4784 + 6197-6198: logits[V] and the greedy token (tie rule of argmax_k); synchronises to return it
    int lm_head_row(const Fp4& w, uint64_t x, uint64_t logits);
    // gen.rs:4168-4534, routed part: ids [t][K] i32, wts [t][K] f32, y[t][H] += sum_j w_j down_e(silu(gate_e x) * up_e x);
    // h2 is scratch [t K][I], dn_ptrs scratch u64 [t][K].  Up to 4 tokens the router runs inside the gate|up launch.
    void moe_run(const MoeW& moe, int t, uint64_t x, uint64_t logits, uint64_t ids, uint64_t wts, uint64_t y, uint64_t h2, uint64_t gu_ptrs,
                 uint64_t dn_ptrs);
    // the same for a batch in which experts repeat (the prefill path's idea, kernels.rs:3322-3384): router_top10, moe_group
    // (combos sorted by expert, tiles of at most four), every tile's slab multiplied once by its rows, acc_combo.
    // eo is scratch [t K][H], perm i32 [t K], tiles i32 [max_tiles][4], n_tiles i32 [1]; max_tiles = min(t K, E) + t K / 4
    void moe_run_grouped(const MoeW& moe, int t, uint64_t x, uint64_t logits, uint64_t ids, uint64_t wts, uint64_t y, uint64_t h2, uint64_t eo,
                         uint64_t gu_ptrs, uint64_t dn_ptrs, uint64_t perm, uint64_t tiles, uint64_t n_tiles);
    static int moe_max_tiles(int combos, int experts) { return (combos < experts ? combos : experts) + combos / 4; }
    // prefill projection: Y[m][rows] = X[m][cols] W^T on the matrix cores, bf16 X
    void gemm(const Fp4& w, int m, uint64_t x_bf16, uint64_t y);
    // the unquantised keeps: y[t][rows] = W[rows][k] x[t][k], f32 x; W bf16 (gemv_bf16_w, kernels.rs:1130-1157) or f32
    // (gemv_b, kernels.rs:97-115: the router projection)
    void bf16_proj(uint64_t w_bf16, int rows, int k, int t, uint64_t x, uint64_t y);
    void f32_proj(uint64_t w_f32, int rows, int k, int t, uint64_t x, uint64_t y);
    void check() { status(); }
    Kernels k;
    Params p;
    KernelGeo geo;

  private:
    Engine(Module m, const KernelGeo* geo);
};

// A captured launch sequence (the reference's CROW_GRAPH path, cuda.rs:113-203): begin() makes the graph's own
// non-blocking stream the current stream and starts capture, launch_v records, end() instantiates, launch() replays.
class Graph {
  public:
    Graph();
    ~Graph();
    Graph(const Graph&) = delete;
    Graph& operator=(const Graph&) = delete;
    void begin();
    void end();
    void launch();
    void sync();

  private:
    void* stream_ = nullptr;
    void* exec_ = nullptr;
    void* prev_ = nullptr;
};

// ---------------------------------------------------------------- CNQ1 container reader
struct TensorInfo {
    std::string name, section, dtype;
    uint64_t offset = 0;  // relative to the blob start
    uint64_t n_values = 0;
    float global_scale = 1.0f;
    std::vector<uint64_t> shape;
};
struct ModelBlock {
    std::string family, model_type, recipe, config_json, generation_config_json, source_repo, source_revision;
};
class Cnq {
  public:
    // Cnq::open_checked (cnq.rs:952-983): every refusal is thrown as Refused with the reference's text
    static Cnq open_checked(const std::string& path);
    // Cnq::open: Panic "[cnq] refused: {path}: {why}"
    static Cnq open(const std::string& path);
    const TensorInfo& find(const std::string& name, const std::string& section) const;  // Panic "tensor not found: {name} [{section}]"
    static uint64_t byte_len(const TensorInfo& t);                                       // cnq.rs:1071-1078
    std::vector<uint8_t> read_bytes(const TensorInfo& t) const;                          // cnq.rs:1122-1128
    std::vector<uint8_t> read_range(const TensorInfo& t, uint64_t rel_off, uint64_t n) const;  // cnq.rs:1129-1135
    const ModelBlock* model() const { return has_model ? &model_block : nullptr; }
    std::string family() const { return has_model ? model_block.family : "FlashNext"; }
    std::string path;
    uint64_t blob_offset = 0, file_len = 0;
    std::vector<TensorInfo> tensors;
    bool has_model = false;
    ModelBlock model_block;

  private:
    std::vector<uint8_t> read_at(uint64_t off, uint64_t n) const;
};
// weights::load_fp4(cnq, name, sec) (weights.rs:26-33): Panic "{name}: expected NVFP4, got {dtype}" for a bf16 / f32 tensor
Fp4 load_fp4(const Cnq& cnq, const std::string& name, const std::string& sec);
std::string sha256_hex(const uint8_t* data, size_t n);

}  // namespace crow

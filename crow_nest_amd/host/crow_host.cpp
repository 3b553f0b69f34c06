// Implementation of crow_host.hpp: everything goes through the C ABI of include/crow_hip.h (no HIP headers here).
#include "crow_host.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <fstream>
#include <sstream>

namespace crow {

// ---------------------------------------------------------------- errors, context
void ck(int rc, const char* what) {
    if (rc == CROW_OK) return;
    char msg[512];
    snprintf(msg, sizeof msg, "HIP error: %s: %s (%d)", what, crow_hip_error_string(rc), rc);
    throw Panic(msg);
}

static bool g_ready = false;
void Ctx::init(int device) {
    ck(crow_hip_init(device), "crow_hip_init");
    g_ready = true;
}
bool Ctx::ready() { return g_ready; }
static void ensure_init() {
    if (!g_ready) Ctx::init(0);
}
void sync() { ck(crow_hip_sync(), "sync"); }
void status() { ck(crow_hip_status(), "kernel status"); }

// ---------------------------------------------------------------- device memory
DevBuf::DevBuf(size_t bytes) : n_(bytes) {
    ensure_init();
    ck(crow_hip_alloc(bytes, &p_), "crow_hip_alloc");
}
DevBuf& DevBuf::operator=(DevBuf&& o) noexcept {
    if (this != &o) {
        if (p_) (void)crow_hip_free(p_);
        p_ = o.p_, n_ = o.n_;
        o.p_ = nullptr, o.n_ = 0;
    }
    return *this;
}
DevBuf::~DevBuf() {
    if (p_) (void)crow_hip_free(p_);  // while a panic unwinds the reference logs and ignores this too (cuda.rs:286-313)
}
void DevBuf::upload(const void* src, size_t bytes, size_t at) {
    if (at + bytes > n_) throw Panic("upload_into: " + std::to_string(bytes) + " B at " + std::to_string(at) + " run off a " + std::to_string(n_) + " B buffer");
    ck(crow_hip_upload((char*)p_ + at, src, bytes), "upload_into");
    sync();  // the source is pageable host memory the caller may free at once
}
void DevBuf::download(void* dst, size_t bytes, size_t at) const {
    if (at + bytes > n_) throw Panic("dtoh: " + std::to_string(bytes) + " B at " + std::to_string(at) + " run off a " + std::to_string(n_) + " B buffer");
    ck(crow_hip_download(dst, (const char*)p_ + at, bytes), "dtoh");
}

// ---------------------------------------------------------------- module, kernel table, launches
crow_fn_t Module::get(const char* name) const {
    crow_fn_t f = nullptr;
    const int rc = crow_hip_module_get(h_, name, &f);
    if (rc == CROW_ERR_KERNEL_MISSING) throw Panic(std::string("kernel missing: ") + name);
    ck(rc, "Module::get");
    return f;
}
void Module::unload() {
    if (h_) ck(crow_hip_module_unload(h_), "Module::unload");
    h_ = nullptr;
}
void set_geo(const KernelGeo& geo) {
    ensure_init();
    ck(crow_hip_set_geo(geo.experts, geo.topk, geo.hidden, geo.inter), "crow_hip_set_geo");
}
Module compile(const KernelGeo* geo) {
    ensure_init();
    crow_module_t h = nullptr;
    ck(crow_hip_module_load(&h), "crow_hip_module_load");
    if (geo) set_geo(*geo);
    return Module(h);
}
Kernels::Kernels(const Module& m) {
    const int n = crow_hip_function_count();
    for (int i = 0; i < n; i++) {
        const char* name = crow_hip_function_name(i);
        map_[name] = m.get(name);
    }
}
crow_fn_t Kernels::f(const std::string& name) const {
    const auto it = map_.find(name);
    if (it == map_.end()) throw Panic("kernel missing: " + name);
    return it->second;
}
Dims launch_dims(const char* name, uint32_t rows, uint32_t k_dim, uint32_t z) {
    crow_dims d{};
    const int rc = crow_hip_launch_dims(name, rows, k_dim, z, &d);
    if (rc == CROW_ERR_KERNEL_MISSING) throw Panic(std::string("kernel missing: ") + name);
    ck(rc, "launch_dims");
    return Dims{d.gx, d.gy, d.gz, d.bx};
}
void launch_v(crow_fn_t f, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, const std::vector<uint64_t>& vals) {
    ck(crow_hip_launch(f, gx, gy, gz, bx, vals.data(), (uint32_t)vals.size(), nullptr), "launch_v");
}
void launch_v(crow_fn_t f, const Dims& d, const std::vector<uint64_t>& vals) { launch_v(f, d.gx, d.gy, d.gz, d.bx, vals); }
void launch_sync(crow_fn_t f, const Dims& d, const std::vector<uint64_t>& vals) {
    launch_v(f, d, vals);
    sync();
}
uint64_t Params::i32(int v) {
    auto it = words_.find(v);
    if (it == words_.end()) {
        DevBuf b(sizeof(int));
        b.upload(&v, sizeof v);
        it = words_.emplace(v, std::move(b)).first;
    }
    return it->second.ptr();
}

// ---------------------------------------------------------------- weights
Nvfp4Matrix Nvfp4Matrix::make(const uint8_t* bytes, size_t len, int rows, int cols, float global_scale) {
    if (cols == 0 || cols % 64 != 0) throw Refused("cpu_nvfp4: " + std::to_string(cols) + " columns are not whole 64-value NVFP4 blocks");
    const size_t want = byte_len(rows, cols);
    if (len != want)
        throw Refused("cpu_nvfp4: [" + std::to_string(rows) + ", " + std::to_string(cols) + "] needs " + std::to_string(want) + " B, got " + std::to_string(len));
    return Nvfp4Matrix{bytes, len, rows, cols, global_scale};
}
ExpertBlock ExpertBlock::make(const Nvfp4Matrix& gate, const Nvfp4Matrix& up, const Nvfp4Matrix& down) {
    const int inter = gate.rows, hidden = gate.cols;
    if (up.rows != inter || up.cols != hidden || down.rows != hidden || down.cols != inter)
        throw Refused("cpu_nvfp4: expert shapes gate [" + std::to_string(gate.rows) + ", " + std::to_string(gate.cols) + "], up [" +
                      std::to_string(up.rows) + ", " + std::to_string(up.cols) + "], down [" + std::to_string(down.rows) + ", " +
                      std::to_string(down.cols) + "] do not fit together");
    return ExpertBlock{gate, up, down, hidden, inter};
}
ExpertBlock ExpertBlock::from_unit(const uint8_t* unit, size_t len, int hidden, int inter, const float (&global_scales)[3]) {
    const size_t gu = Nvfp4Matrix::byte_len(inter, hidden), dn = Nvfp4Matrix::byte_len(hidden, inter);
    if (len != 2 * gu + dn)
        throw Refused("cpu_nvfp4: expert unit H " + std::to_string(hidden) + " I " + std::to_string(inter) + " needs " + std::to_string(2 * gu + dn) +
                      " B, got " + std::to_string(len));
    return make(Nvfp4Matrix::make(unit, gu, inter, hidden, global_scales[0]), Nvfp4Matrix::make(unit + gu, gu, inter, hidden, global_scales[1]),
                Nvfp4Matrix::make(unit + 2 * gu, dn, hidden, inter, global_scales[2]));
}
static void repack_into(uint64_t raw_dev, int rows, int cols, uint64_t dst_dev) {
    ck(crow_hip_repack_nvfp4((const void*)(uintptr_t)raw_dev, (uint32_t)rows, (uint32_t)cols, (void*)(uintptr_t)dst_dev), "crow_hip_repack_nvfp4");
}
Fp4 load_fp4(const Nvfp4Matrix& m) {
    ensure_init();
    DevBuf raw(m.len);
    raw.upload(m.bytes, m.len);
    Fp4 out;
    out.w = DevBuf(crow_hip_tiled_bytes((uint32_t)m.rows, (uint32_t)m.cols));
    repack_into(raw.ptr(), m.rows, m.cols, out.w.ptr());
    out.gs = DevBuf(sizeof(float));
    out.gs.upload(&m.global_scale, sizeof(float));
    out.rows = m.rows, out.cols = m.cols;
    sync();  // the raw copy is freed when this returns
    status();
    return out;
}
QuantizedNvfp4 quantize_nvfp4(const float* values, size_t n_values) {
    ensure_init();
    if (n_values % 64 != 0) throw Panic("assertion failed: values.len() % 64 == 0");
    QuantizedNvfp4 q;
    q.blocks.resize(n_values / 64 * 36);
    if (n_values == 0) return q;
    DevBuf v(n_values * sizeof(float)), b(q.blocks.size()), g(sizeof(float));
    v.upload(values, n_values * sizeof(float));
    ck(crow_hip_quantize_nvfp4((const float*)(uintptr_t)v.ptr(), n_values, (void*)(uintptr_t)b.ptr(), (float*)(uintptr_t)g.ptr()), "crow_hip_quantize_nvfp4");
    b.download(q.blocks.data(), q.blocks.size());
    g.download(&q.global_scale, sizeof(float));
    status();
    return q;
}
MlpW load_expert_block(const ExpertBlock& e) {
    MlpW m;
    m.gate = load_fp4(e.gate), m.up = load_fp4(e.up), m.down = load_fp4(e.down);
    return m;
}
std::vector<float> dequant(const Fp4& w) {
    const size_t n = (size_t)w.rows * w.cols;
    DevBuf out(n * sizeof(float));
    ck(crow_hip_dequant_tiled((const void*)(uintptr_t)w.w.ptr(), (const float*)(uintptr_t)w.gs.ptr(), (uint32_t)w.rows, (uint32_t)w.cols,
                              (float*)(uintptr_t)out.ptr()),
       "crow_hip_dequant_tiled");
    std::vector<float> host(n);
    out.download(host.data(), n * sizeof(float));
    return host;
}
ExpertSlabs load_expert_slabs(const uint8_t* data, size_t len, int experts, int rows, int cols, float global_scale) {
    ensure_init();
    if (cols == 0 || cols % 64 != 0) throw Refused("cpu_nvfp4: " + std::to_string(cols) + " columns are not whole 64-value NVFP4 blocks");
    const size_t per = Nvfp4Matrix::byte_len(rows, cols);
    if (len != (size_t)experts * per)
        throw Refused("cpu_nvfp4: [" + std::to_string(experts) + "][" + std::to_string(rows) + ", " + std::to_string(cols) + "] needs " +
                      std::to_string((size_t)experts * per) + " B, got " + std::to_string(len));
    ExpertSlabs s;
    s.experts = experts, s.rows = rows, s.cols = cols;
    s.slab_bytes = crow_hip_tiled_bytes((uint32_t)rows, (uint32_t)cols);
    DevBuf raw(len);
    raw.upload(data, len);
    s.w = DevBuf((size_t)experts * s.slab_bytes);
    for (int e = 0; e < experts; e++) repack_into(raw.ptr() + (uint64_t)e * per, rows, cols, s.ptr(e));
    s.gs = DevBuf(sizeof(float));
    s.gs.upload(&global_scale, sizeof(float));
    sync();
    status();
    return s;
}
MoeW make_moe(ExpertSlabs gate_up, ExpertSlabs down) {
    if (gate_up.experts != down.experts) throw Panic("moe: gate_up holds " + std::to_string(gate_up.experts) + " experts, down " + std::to_string(down.experts));
    std::vector<uint64_t> table((size_t)gate_up.experts * 2);
    for (int e = 0; e < gate_up.experts; e++) table[2 * e] = gate_up.ptr(e), table[2 * e + 1] = down.ptr(e);
    MoeW m;
    m.table = DevBuf(table.size() * sizeof(uint64_t));
    m.table.upload(table.data(), table.size() * sizeof(uint64_t));
    m.gate_up = std::move(gate_up);
    m.down = std::move(down);
    return m;
}

// ---------------------------------------------------------------- the engine's dispatch
Engine::Engine(Module m, const KernelGeo* g) : k(m), geo(g ? *g : KernelGeo{}) {}
Engine::Engine(const KernelGeo* g) : Engine(compile(g), g) {}

void Engine::dense_proj(const Fp4& w, int t, uint64_t x, uint64_t y, bool x_bf16) {
    const uint32_t rows = (uint32_t)w.rows, kd = (uint32_t)w.cols;
    if (t == 1 && !x_bf16) {
        launch_v(k.f("gemv_nvfp4_w"), launch_dims("gemv_nvfp4_w", rows, kd), {w.w.ptr(), x, w.gs.ptr(), y, p.i32(w.cols), p.i32(w.rows)});
    } else if (t <= NVFP4_MMAX) {
        proj_m(w, t, x, y, x_bf16);
    } else if (x_bf16) {
        gemm(w, t, x, y);
    } else {
        launch_v(k.f("gemv_fp4_b"), launch_dims("gemv_fp4_b", rows, kd, (uint32_t)t), {w.w.ptr(), x, w.gs.ptr(), y, p.i32(w.cols), p.i32(w.rows), p.i32(t)});
    }
}
void Engine::proj_m(const Fp4& w, int m, uint64_t x, uint64_t y, bool x_bf16) {
    if (m < 1 || m > NVFP4_MMAX) throw Panic("proj_m: M = " + std::to_string(m) + " is outside 1..=" + std::to_string(NVFP4_MMAX));
    const char* name = x_bf16 ? "gemv_nvfp4_wm_bf16" : "gemv_nvfp4_wm";
    launch_v(k.f(name), launch_dims(name, (uint32_t)w.rows, (uint32_t)w.cols, (uint32_t)m), {w.w.ptr(), x, w.gs.ptr(), y, p.i32(w.cols), p.i32(w.rows), p.i32(m)});
}
void Engine::gate_up(const MlpW& mlp, int t, uint64_t x, uint64_t h, bool x_bf16) {
    const int inter = mlp.gate.rows, kd = mlp.gate.cols;
    if (mlp.up.rows != inter || mlp.up.cols != kd) throw Panic("gate_up: gate and up differ in shape");
    if (t < 1 || t > NVFP4_MMAX) throw Panic("gate_up: " + std::to_string(t) + " rows are outside 1..=" + std::to_string(NVFP4_MMAX));
    if (t == 1) {
        const char* name = x_bf16 ? "gemv_nvfp4_gu_bf16" : "gemv_nvfp4_gu";
        launch_v(k.f(name), launch_dims(name, (uint32_t)inter, (uint32_t)kd),
                 {mlp.gate.w.ptr(), mlp.up.w.ptr(), x, mlp.gate.gs.ptr(), mlp.up.gs.ptr(), h, p.i32(kd), p.i32(inter)});
    } else {
        const char* name = x_bf16 ? "gemv_nvfp4_gum_bf16" : "gemv_nvfp4_gum";
        launch_v(k.f(name), launch_dims(name, (uint32_t)inter, (uint32_t)kd, (uint32_t)t),
                 {mlp.gate.w.ptr(), mlp.up.w.ptr(), x, mlp.gate.gs.ptr(), mlp.up.gs.ptr(), h, p.i32(kd), p.i32(inter), p.i32(t)});
    }
}
void Engine::dense_ffn_w(const MlpW& mlp, uint64_t x, int t, uint64_t h, uint64_t y, bool x_bf16) {
    gate_up(mlp, t, x, h, x_bf16);
    dense_proj(mlp.down, t, h, y);
}
int Engine::lm_head_row(const Fp4& w, uint64_t x, uint64_t logits) {
    DevBuf idx(sizeof(int));
    launch_v(k.f("gemv_nvfp4_w_argmax"), launch_dims("gemv_nvfp4_w_argmax", (uint32_t)w.rows, (uint32_t)w.cols),
             {w.w.ptr(), x, w.gs.ptr(), logits, p.i32(w.cols), p.i32(w.rows), idx.ptr()});
    int out = -1;
    idx.download(&out, sizeof out);
    return out;
}
void Engine::moe_run(const MoeW& moe, int t, uint64_t x, uint64_t logits, uint64_t ids, uint64_t wts, uint64_t y, uint64_t h2, uint64_t gu_ptrs,
                     uint64_t dn_ptrs) {
    const int hdim = geo.hidden, inter = geo.inter, topk = geo.topk;
    if (moe.gate_up.rows != 2 * inter || moe.gate_up.cols != hdim || moe.down.rows != hdim || moe.down.cols != inter || moe.gate_up.experts != geo.experts)
        throw Panic("moe_run: the expert tensors do not match the geometry");
    const uint32_t combos = (uint32_t)(t * topk);
    if (t <= 4) {  // the router inside the gate|up launch
        launch_v(k.f("moe_route_gate_up_silu"), launch_dims("moe_route_gate_up_silu", (uint32_t)inter, (uint32_t)hdim, combos),
                 {logits, moe.table.ptr(), x, moe.gate_up.gs.ptr(), h2, ids, wts, dn_ptrs, p.i32(hdim), p.i32(hdim), p.i32(inter)});
    } else {
        launch_v(k.f("router_top10"), launch_dims("router_top10", 1, 64, (uint32_t)t), {logits, 0, ids, wts, gu_ptrs, dn_ptrs, moe.table.ptr(), 0, 0, 0});
        launch_v(k.f("moe_gate_up_silu"), launch_dims("moe_gate_up_silu", (uint32_t)inter, (uint32_t)hdim, combos),
                 {gu_ptrs, x, moe.gate_up.gs.ptr(), h2, p.i32(hdim), p.i32(topk), p.i32(hdim), p.i32(inter)});
    }
    launch_v(k.f("moe_down_combine"), launch_dims("moe_down_combine", (uint32_t)hdim, (uint32_t)inter, (uint32_t)t),
             {dn_ptrs, h2, moe.down.gs.ptr(), wts, y, p.i32(inter), p.i32(hdim)});
}
void Engine::moe_run_grouped(const MoeW& moe, int t, uint64_t x, uint64_t logits, uint64_t ids, uint64_t wts, uint64_t y, uint64_t h2, uint64_t eo,
                             uint64_t gu_ptrs, uint64_t dn_ptrs, uint64_t perm, uint64_t tiles, uint64_t n_tiles) {
    const int hdim = geo.hidden, inter = geo.inter, topk = geo.topk;
    if (moe.gate_up.rows != 2 * inter || moe.gate_up.cols != hdim || moe.down.rows != hdim || moe.down.cols != inter || moe.gate_up.experts != geo.experts)
        throw Panic("moe_run_grouped: the expert tensors do not match the geometry");
    const int combos = t * topk, max_tiles = moe_max_tiles(combos, geo.experts);
    launch_v(k.f("router_top10"), launch_dims("router_top10", 1, 64, (uint32_t)t), {logits, 0, ids, wts, gu_ptrs, dn_ptrs, moe.table.ptr(), 0, 0, 0});
    launch_v(k.f("moe_group"), launch_dims("moe_group", 1, 64, (uint32_t)combos), {ids, p.i32(combos), perm, tiles, n_tiles, p.i32(max_tiles)});
    launch_v(k.f("moe_gate_up_silu_grouped"), launch_dims("moe_gate_up_silu_grouped", (uint32_t)inter, (uint32_t)hdim, (uint32_t)max_tiles),
             {tiles, n_tiles, perm, moe.table.ptr(), x, moe.gate_up.gs.ptr(), h2, p.i32(hdim), p.i32(topk), p.i32(hdim), p.i32(inter)});
    launch_v(k.f("moe_down_grouped"), launch_dims("moe_down_grouped", (uint32_t)hdim, (uint32_t)inter, (uint32_t)max_tiles),
             {tiles, n_tiles, perm, moe.table.ptr(), h2, moe.down.gs.ptr(), eo, p.i32(inter), p.i32(hdim)});
    launch_v(k.f("acc_combo"), launch_dims("acc_combo", (uint32_t)hdim, 1, (uint32_t)t), {eo, wts, y});
}
void Engine::bf16_proj(uint64_t w_bf16, int rows, int kd, int t, uint64_t x, uint64_t y) {
    launch_v(k.f("gemv_bf16_w"), launch_dims("gemv_bf16_w", (uint32_t)rows, (uint32_t)kd, (uint32_t)t), {w_bf16, x, y, p.i32(kd), p.i32(rows)});
}
void Engine::f32_proj(uint64_t w_f32, int rows, int kd, int t, uint64_t x, uint64_t y) {
    launch_v(k.f("gemv_b"), launch_dims("gemv_b", (uint32_t)rows, (uint32_t)kd, (uint32_t)t), {w_f32, x, y, p.i32(kd), p.i32(rows)});
}
void Engine::gemm(const Fp4& w, int m, uint64_t x_bf16, uint64_t y) {
    const char* name = crow_hip_gemm_kernel((uint32_t)w.rows, (uint32_t)m);
    launch_v(k.f(name), launch_dims(name, (uint32_t)w.rows, (uint32_t)w.cols, (uint32_t)m), {w.w.ptr(), x_bf16, w.gs.ptr(), y, p.i32(w.cols), p.i32(w.rows), p.i32(m)});
}

// ---------------------------------------------------------------- graph capture
Graph::Graph() {
    ensure_init();
    ck(crow_hip_stream_create(&stream_), "crow_hip_stream_create");
}
Graph::~Graph() {
    if (exec_) (void)crow_hip_graph_exec_destroy(exec_);
    if (crow_hip_cur_stream() == stream_) crow_hip_set_stream(nullptr);
    if (stream_) (void)crow_hip_stream_destroy(stream_);
}
void Graph::begin() {
    prev_ = crow_hip_cur_stream();
    ck(crow_hip_begin_capture(stream_), "crow_hip_begin_capture");
}
void Graph::end() {
    const int rc = crow_hip_end_capture_instantiate(stream_, &exec_);
    crow_hip_set_stream(prev_);  // launches after the capture go where they went before it
    ck(rc, "crow_hip_end_capture_instantiate");
}
void Graph::launch() { ck(crow_hip_launch_graph(exec_, stream_), "crow_hip_launch_graph"); }
void Graph::sync() {  // the graph runs on its own non-blocking stream
    void* cur = crow_hip_cur_stream();
    crow_hip_set_stream(stream_);
    const int rc = crow_hip_sync();
    crow_hip_set_stream(cur);
    ck(rc, "sync");
}

// ---------------------------------------------------------------- sha256 (FIPS 180-4), for the index checks of the container
namespace {
struct Sha256 {
    uint32_t h[8] = {0x6a09e667u, 0xbb67ae85u, 0x3c6ef372u, 0xa54ff53au, 0x510e527fu, 0x9b05688cu, 0x1f83d9abu, 0x5be0cd19u};
    uint8_t buf[64];
    size_t fill = 0;
    uint64_t total = 0;
    static uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }
    void block(const uint8_t* p) {
        static const uint32_t K[64] = {
            0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01, 0x243185be,
            0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa,
            0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967, 0x27b70a85,
            0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85, 0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3,
            0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f,
            0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
        uint32_t w[64];
        for (int i = 0; i < 16; i++) w[i] = (uint32_t)p[4 * i] << 24 | (uint32_t)p[4 * i + 1] << 16 | (uint32_t)p[4 * i + 2] << 8 | p[4 * i + 3];
        for (int i = 16; i < 64; i++) {
            const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3), s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
            w[i] = w[i - 16] + s0 + w[i - 7] + s1;
        }
        uint32_t a = h[0], b = h[1], c = h[2], d = h[3], e = h[4], f = h[5], g = h[6], hh = h[7];
        for (int i = 0; i < 64; i++) {
            const uint32_t t1 = hh + (rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25)) + ((e & f) ^ (~e & g)) + K[i] + w[i];
            const uint32_t t2 = (rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22)) + ((a & b) ^ (a & c) ^ (b & c));
            hh = g, g = f, f = e, e = d + t1, d = c, c = b, b = a, a = t1 + t2;
        }
        h[0] += a, h[1] += b, h[2] += c, h[3] += d, h[4] += e, h[5] += f, h[6] += g, h[7] += hh;
    }
    void update(const uint8_t* p, size_t n) {
        total += n;
        while (n > 0) {
            const size_t take = std::min(n, 64 - fill);
            memcpy(buf + fill, p, take);
            fill += take, p += take, n -= take;
            if (fill == 64) block(buf), fill = 0;
        }
    }
    std::string hex() {
        const uint64_t bits = total * 8;
        const uint8_t one = 0x80, zero = 0;
        update(&one, 1);
        while (fill != 56) update(&zero, 1);
        uint8_t len[8];
        for (int i = 0; i < 8; i++) len[i] = (uint8_t)(bits >> (56 - 8 * i));
        update(len, 8);
        char out[65];
        for (int i = 0; i < 8; i++) snprintf(out + 8 * i, 9, "%08x", h[i]);
        return std::string(out, 64);
    }
};
}  // namespace
std::string sha256_hex(const uint8_t* data, size_t n) {
    Sha256 s;
    s.update(data, n);
    return s.hex();
}

// ---------------------------------------------------------------- a small JSON reader for the container index
namespace {
struct Json {
    enum Kind { Null, Bool, Num, Str, Arr, Obj } kind = Null;
    bool b = false;
    double num = 0.0;
    bool is_int = false;
    long long i = 0;
    std::string s, raw;  // raw: the number's text, for messages that quote it
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj;
    const Json* get(const char* key) const {
        if (kind != Obj) return nullptr;
        for (const auto& kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
    bool is_str() const { return kind == Str; }
    std::string dump() const {  // for refusal texts that quote a value
        switch (kind) {
            case Null: return "null";
            case Bool: return b ? "true" : "false";
            case Num: return raw;
            case Str: return "\"" + s + "\"";
            case Arr: return "[...]";
            default: return "{...}";
        }
    }
};
struct JsonParser {
    const char* p;
    const char* end;
    [[noreturn]] void fail(const std::string& what) const { throw Refused("index json: " + what + " at byte " + std::to_string(p - begin)); }
    const char* begin;
    JsonParser(const char* b, const char* e) : p(b), end(e), begin(b) {}
    void ws() {
        while (p < end && (*p == ' ' || *p == '\n' || *p == '\r' || *p == '\t')) p++;
    }
    static void utf8(std::string& out, unsigned cp) {
        if (cp < 0x80) out += (char)cp;
        else if (cp < 0x800) out += (char)(0xC0 | cp >> 6), out += (char)(0x80 | (cp & 0x3F));
        else if (cp < 0x10000) out += (char)(0xE0 | cp >> 12), out += (char)(0x80 | ((cp >> 6) & 0x3F)), out += (char)(0x80 | (cp & 0x3F));
        else out += (char)(0xF0 | cp >> 18), out += (char)(0x80 | ((cp >> 12) & 0x3F)), out += (char)(0x80 | ((cp >> 6) & 0x3F)), out += (char)(0x80 | (cp & 0x3F));
    }
    unsigned hex4() {
        if (end - p < 4) fail("short \\u escape");
        unsigned v = 0;
        for (int i = 0; i < 4; i++) {
            const char c = *p++;
            v = v * 16 + (c >= '0' && c <= '9' ? c - '0' : c >= 'a' && c <= 'f' ? c - 'a' + 10 : c >= 'A' && c <= 'F' ? c - 'A' + 10 : (fail("bad \\u escape"), 0));
        }
        return v;
    }
    std::string str() {
        if (p >= end || *p != '"') fail("expected a string");
        p++;
        std::string out;
        while (true) {
            if (p >= end) fail("unterminated string");
            const char c = *p++;
            if (c == '"') return out;
            if (c != '\\') {
                out += c;
                continue;
            }
            if (p >= end) fail("unterminated escape");
            const char e = *p++;
            switch (e) {
                case '"': out += '"'; break;
                case '\\': out += '\\'; break;
                case '/': out += '/'; break;
                case 'b': out += '\b'; break;
                case 'f': out += '\f'; break;
                case 'n': out += '\n'; break;
                case 'r': out += '\r'; break;
                case 't': out += '\t'; break;
                case 'u': {
                    unsigned cp = hex4();
                    if (cp >= 0xD800 && cp < 0xDC00 && end - p >= 6 && p[0] == '\\' && p[1] == 'u') {
                        p += 2;
                        const unsigned lo = hex4();
                        cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                    }
                    utf8(out, cp);
                    break;
                }
                default: fail("bad escape");
            }
        }
    }
    Json value(int depth = 0) {
        if (depth > 64) fail("nesting too deep");
        ws();
        if (p >= end) fail("unexpected end");
        Json j;
        const char c = *p;
        if (c == '{') {
            p++;
            j.kind = Json::Obj;
            ws();
            if (p < end && *p == '}') return p++, j;
            while (true) {
                ws();
                std::string key = str();
                ws();
                if (p >= end || *p != ':') fail("expected ':'");
                p++;
                j.obj.emplace_back(std::move(key), value(depth + 1));
                ws();
                if (p < end && *p == ',') {
                    p++;
                    continue;
                }
                if (p < end && *p == '}') return p++, j;
                fail("expected ',' or '}'");
            }
        }
        if (c == '[') {
            p++;
            j.kind = Json::Arr;
            ws();
            if (p < end && *p == ']') return p++, j;
            while (true) {
                j.arr.push_back(value(depth + 1));
                ws();
                if (p < end && *p == ',') {
                    p++;
                    continue;
                }
                if (p < end && *p == ']') return p++, j;
                fail("expected ',' or ']'");
            }
        }
        if (c == '"') {
            j.kind = Json::Str;
            j.s = str();
            return j;
        }
        if (end - p >= 4 && !strncmp(p, "true", 4)) return p += 4, j.kind = Json::Bool, j.b = true, j;
        if (end - p >= 5 && !strncmp(p, "false", 5)) return p += 5, j.kind = Json::Bool, j.b = false, j;
        if (end - p >= 4 && !strncmp(p, "null", 4)) return p += 4, j;
        const char* s = p;
        if (p < end && *p == '-') p++;
        bool integral = true;
        while (p < end && ((*p >= '0' && *p <= '9') || *p == '.' || *p == 'e' || *p == 'E' || *p == '+' || *p == '-')) {
            if (*p == '.' || *p == 'e' || *p == 'E') integral = false;
            p++;
        }
        if (p == s) fail("unexpected character");
        j.kind = Json::Num;
        j.raw.assign(s, p);
        j.num = strtod(j.raw.c_str(), nullptr);
        j.is_int = integral;
        if (integral) j.i = strtoll(j.raw.c_str(), nullptr, 10);
        return j;
    }
};
const char* const CNQ45M_INDEX_SHA256 = "a21afc43203d983e46be5dd378ac5fb34581ab31fb5a0f6e8093d4730078c4ba";  // cnq.rs:86
const unsigned long CNQ45M_INDEX_LEN = 473528;                                                                 // cnq.rs:89
const char* const V1_REFUSAL = "CNQ index v1 is only accepted for the Flash-Next CNQ4.5-M container of record";

std::string req_str(const Json* v, const char* what) {
    if (!v || !v->is_str()) throw Refused(std::string("CNQ index v2: `") + what + "` missing or not a string");
    return v->s;
}
ModelBlock parse_model_block(const Json& index) {  // cnq.rs:196-239
    const Json* m = index.get("model");
    if (!m || m->kind != Json::Obj) throw Refused("CNQ index v2 without a `model` block");
    ModelBlock b;
    b.config_json = req_str(m->get("config_json"), "model.config_json");
    b.generation_config_json = req_str(m->get("generation_config_json"), "model.generation_config_json");
    const std::pair<const char*, const std::string*> stored[2] = {{"config_json", &b.config_json}, {"generation_config_json", &b.generation_config_json}};
    for (const auto& st : stored) {
        const std::string key = std::string(st.first) + "_sha256";
        const std::string want = req_str(m->get(key.c_str()), ("model." + key).c_str());
        const std::string got = sha256_hex((const uint8_t*)st.second->data(), st.second->size());
        if (got != want)
            throw Refused(std::string("CNQ index v2: model.") + st.first + " hashes to " + got + ", the index records " + want + " - the stored config was altered");
    }
    const Json* src = m->get("source");
    static const Json none;
    if (!src || src->kind != Json::Obj) src = &none;
    b.family = req_str(m->get("family"), "model.family");
    b.model_type = req_str(m->get("model_type"), "model.model_type");
    b.recipe = req_str(index.get("recipe"), "recipe");
    b.source_repo = req_str(src->get("repo"), "model.source.repo");
    b.source_revision = req_str(src->get("revision"), "model.source.revision");
    return b;
}
}  // namespace

// ---------------------------------------------------------------- the container
Cnq Cnq::open_checked(const std::string& path) {
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) throw Refused("cannot open " + path);
    const uint64_t file_len = (uint64_t)f.tellg();
    if (file_len < 20) throw Refused(std::to_string(file_len) + " B is too small to be a CNQ1 container");
    uint8_t magic[4];
    f.seekg(0);
    f.read((char*)magic, 4);
    if (memcmp(magic, "CNQ1", 4) != 0) {
        std::ostringstream o;
        o << "magic is [" << (int)magic[0] << ", " << (int)magic[1] << ", " << (int)magic[2] << ", " << (int)magic[3] << "], not CNQ1";
        throw Refused(o.str());
    }
    uint8_t lb[8];
    f.seekg((std::streamoff)(file_len - 8));
    f.read((char*)lb, 8);
    uint64_t idx_len = 0;
    for (int i = 7; i >= 0; i--) idx_len = idx_len << 8 | lb[i];
    if (idx_len == 0 || idx_len + 20 > file_len) throw Refused("index length " + std::to_string(idx_len) + " does not fit a " + std::to_string(file_len) + " B file");
    std::vector<char> ib(idx_len);
    f.seekg((std::streamoff)(file_len - 8 - idx_len));
    f.read(ib.data(), (std::streamsize)idx_len);
    if (!f) throw Refused("short read of the index of " + path);
    JsonParser jp(ib.data(), ib.data() + ib.size());
    const Json index = jp.value();

    Cnq c;
    c.path = path;
    c.file_len = file_len;
    // classify_index, cnq.rs:175-195: the v1 container of record, or an index v2; anything else is refused
    const Json* fv = index.get("format_version");
    if (!fv || fv->kind == Json::Null) {
        const Json* v = index.get("version");
        if (v && v->kind != Json::Null && !(v->kind == Json::Num && v->is_int && v->i == 1))
            throw Refused("CNQ index `version` " + v->dump() + " without a `format_version` - not an index this engine reads");
        const std::string got = sha256_hex((const uint8_t*)ib.data(), ib.size());
        if (got != CNQ45M_INDEX_SHA256)
            throw Refused(std::string(V1_REFUSAL) + " (index sha256 " + got + ", " + std::to_string(ib.size()) + " B; of record " + CNQ45M_INDEX_SHA256 + ", " +
                          std::to_string(CNQ45M_INDEX_LEN) + " B) - re-convert the checkpoint: the converter writes index v2, which carries the model's config");
    } else if (fv->kind == Json::Num && fv->is_int && fv->i == 2) {
        c.model_block = parse_model_block(index);
        c.has_model = true;
    } else {
        throw Refused("CNQ index format_version " + fv->dump() + " is not one this engine reads (it reads 2, and v1 only for the container of record)");
    }
    const Json* bo = index.get("blob_offset");
    if (!bo || bo->kind != Json::Num || !bo->is_int || bo->i < 0) throw Refused("index has no blob_offset");
    c.blob_offset = (uint64_t)bo->i;
    // parse_tensor_index, cnq.rs:715-733
    if (const Json* ts = index.get("tensors"); ts && ts->kind == Json::Arr)
        for (const Json& t : ts->arr) {
            TensorInfo ti;
            const Json *n = t.get("name"), *s = t.get("section"), *d = t.get("dtype"), *o = t.get("offset"), *nv = t.get("n_values");
            if (!n || !n->is_str() || !s || !s->is_str() || !d || !d->is_str() || !o || o->kind != Json::Num || !nv || nv->kind != Json::Num)
                throw Refused("tensor index entry without name / section / dtype / offset / n_values");
            ti.name = n->s, ti.section = s->s, ti.dtype = d->s;
            ti.offset = (uint64_t)o->i, ti.n_values = (uint64_t)nv->i;
            const Json* gs = t.get("global_scale");
            ti.global_scale = gs && gs->kind == Json::Num ? (float)gs->num : 1.0f;
            if (const Json* sh = t.get("shape"); sh && sh->kind == Json::Arr)
                for (const Json& v : sh->arr) ti.shape.push_back((uint64_t)v.i);
            c.tensors.push_back(std::move(ti));
        }
    return c;
}
Cnq Cnq::open(const std::string& path) {
    try {
        return open_checked(path);
    } catch (const Refused& why) {
        throw Panic("[cnq] refused: " + path + ": " + why.what());
    }
}
const TensorInfo& Cnq::find(const std::string& name, const std::string& section) const {
    for (const auto& t : tensors)
        if (t.name == name && t.section == section) return t;
    throw Panic("tensor not found: " + name + " [" + section + "]");
}
uint64_t Cnq::byte_len(const TensorInfo& t) {
    if (t.dtype == "bf16") return t.n_values * 2;
    if (t.dtype == "i64") return t.n_values * 8;
    if (t.dtype == "f32") return t.n_values * 4;
    return (t.n_values + 63) / 64 * 36;  // nvfp4
}
std::vector<uint8_t> Cnq::read_at(uint64_t off, uint64_t n) const {
    if (n > file_len - 8 || off > file_len - 8 - n) throw Refused("read of " + std::to_string(n) + " B at " + std::to_string(off) + " runs off the payload of a " + std::to_string(file_len) + " B container");
    std::ifstream f(path, std::ios::binary);
    std::vector<uint8_t> out(n);
    f.seekg((std::streamoff)off);
    f.read((char*)out.data(), (std::streamsize)n);
    if (!f) throw Panic(path + ": short read (" + std::to_string(f.gcount()) + " of " + std::to_string(n) + " B at " + std::to_string(off) + ")");
    return out;
}
std::vector<uint8_t> Cnq::read_bytes(const TensorInfo& t) const { return read_at(blob_offset + t.offset, byte_len(t)); }
std::vector<uint8_t> Cnq::read_range(const TensorInfo& t, uint64_t rel_off, uint64_t n) const { return read_at(blob_offset + t.offset + rel_off, n); }

Fp4 load_fp4(const Cnq& cnq, const std::string& name, const std::string& sec) {
    const TensorInfo& t = cnq.find(name, sec);
    if (t.dtype == "bf16" || t.dtype == "f32") throw Panic(name + ": expected NVFP4, got " + t.dtype);
    if (t.shape.size() != 2 || t.shape[0] * t.shape[1] != t.n_values) throw Refused(name + ": the index entry's shape is not a matrix of " + std::to_string(t.n_values) + " values");
    const std::vector<uint8_t> bytes = cnq.read_bytes(t);
    return load_fp4(Nvfp4Matrix::make(bytes.data(), bytes.size(), (int)t.shape[0], (int)t.shape[1], t.global_scale));
}

}  // namespace crow

// Test driver for the C++ host layer (crow_nest_amd/host): each subcommand runs one caller of the hot path the way the
// reference's own tests drive theirs - load weights, call the engine function, hand the result back - on files the
// Python tests write and check against the CPU oracle.  No oracle, no Python, no torch in this process.
//
//   missing                     launch_dims on an unknown name -> prints the panic text (no GPU needed)
//   matrix-checks               Nvfp4Matrix::make refusals -> prints the texts (no GPU needed)
//   cnq-list <file>             the container's table, one line per tensor (no GPU needed)
//   cnq-refuse <file>           prints the text open_checked refuses the file with (no GPU needed)
//   cnq-dequant <file> <dir>    every 2-D NVFP4 tensor: load_fp4(cnq, name, sec), dequantise, write <dir>/<index>.f32
//   dense <dir>                 meta: H I R T xbf16; dense_ffn_w (T <= 4) -> h.bin, y.bin; dense_proj(gate) on f32 x -> gate_y.bin;
//                               T = 1, f32 x: the step captured in a Graph and replayed -> y_graph.bin
//   head <dir>                  meta: V K; lm_head_row -> logits.bin, prints the token
//   moe <dir>                   meta: E topk H I T; moe_run -> ids.bin, wts.bin, y.bin
//   gemm <dir>                  meta: rows cols M; Engine::gemm -> y.bin
//   moe-grouped <dir>           meta as moe; moe_run_grouped -> ids.bin, wts.bin, y.bin
//   keeps <dir>                 meta: rows k t; bf16_proj, f32_proj -> y_bf16.bin, y_f32.bin
//   panics                      Kernels::f on an unknown name, proj_m outside 1..=4 -> prints the texts
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <sstream>

#include "../../crow_nest_amd/host/crow_host.hpp"

using namespace crow;

static std::vector<uint8_t> slurp(const std::string& path) {
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) throw std::runtime_error("cannot open " + path);
    std::vector<uint8_t> b((size_t)f.tellg());
    f.seekg(0);
    f.read((char*)b.data(), (std::streamsize)b.size());
    return b;
}
static void spit(const std::string& path, const void* p, size_t n) {
    std::ofstream f(path, std::ios::binary);
    f.write((const char*)p, (std::streamsize)n);
    if (!f) throw std::runtime_error("cannot write " + path);
}
static std::vector<long> meta(const std::string& dir) {
    std::ifstream f(dir + "/meta.txt");
    std::vector<long> v;
    long x;
    while (f >> x) v.push_back(x);
    return v;
}
static DevBuf to_dev(const std::vector<uint8_t>& b) {
    DevBuf d(b.size());
    d.upload(b.data(), b.size());
    return d;
}
static void from_dev(const DevBuf& d, const std::string& path) {
    std::vector<uint8_t> b(d.bytes());
    d.download(b.data(), b.size());
    spit(path, b.data(), b.size());
}
static Fp4 load(const std::string& path, int rows, int cols, float gs) {
    const std::vector<uint8_t> b = slurp(path);
    return load_fp4(Nvfp4Matrix::make(b.data(), b.size(), rows, cols, gs));
}

static int cnq_list(const std::string& file) {
    const Cnq c = Cnq::open(file);
    const ModelBlock* m = c.model();
    printf("family=%s model_type=%s recipe=%s repo=%s revision=%s blob_offset=%llu tensors=%zu\n", c.family().c_str(), m ? m->model_type.c_str() : "",
           m ? m->recipe.c_str() : "", m ? m->source_repo.c_str() : "", m ? m->source_revision.c_str() : "", (unsigned long long)c.blob_offset, c.tensors.size());
    for (const auto& t : c.tensors) {
        printf("%s|%s|%s|%llu|%llu|%llu|%.9g|", t.name.c_str(), t.section.c_str(), t.dtype.c_str(), (unsigned long long)t.offset, (unsigned long long)t.n_values,
               (unsigned long long)Cnq::byte_len(t), (double)t.global_scale);
        for (size_t i = 0; i < t.shape.size(); i++) printf("%s%llu", i ? "," : "", (unsigned long long)t.shape[i]);
        printf("\n");
    }
    try {
        c.find("lm_head.weight", "no-such-section");
    } catch (const Panic& e) {
        printf("find: %s\n", e.what());
    }
    return 0;
}

static int cnq_dequant(const std::string& file, const std::string& dir) {
    const Cnq c = Cnq::open(file);
    for (size_t i = 0; i < c.tensors.size(); i++) {
        const TensorInfo& t = c.tensors[i];
        if (t.dtype == "bf16" || t.dtype == "f32" || t.dtype == "i64" || t.shape.size() != 2) continue;
        const Fp4 w = load_fp4(c, t.name, t.section);
        const std::vector<float> v = dequant(w);
        spit(dir + "/" + std::to_string(i) + ".f32", v.data(), v.size() * sizeof(float));
    }
    try {
        load_fp4(c, "model.language_model.layers.0.linear_attn.A_log", "text");
    } catch (const Panic& e) {
        printf("load_fp4: %s\n", e.what());
    }
    status();
    return 0;
}

static int dense(const std::string& dir) {
    const std::vector<long> m = meta(dir);
    const int H = (int)m.at(0), I = (int)m.at(1), R = (int)m.at(2), T = (int)m.at(3);
    const bool xbf16 = m.at(4) != 0;
    const std::vector<uint8_t> gsb = slurp(dir + "/gs.bin");
    const float* gs = (const float*)gsb.data();
    Engine eng;
    MlpW mlp{load(dir + "/gate.bin", I, H, gs[0]), load(dir + "/up.bin", I, H, gs[1]), load(dir + "/down.bin", R, I, gs[2])};
    DevBuf x = to_dev(slurp(dir + "/x.bin"));
    DevBuf h((size_t)T * I * 4), y((size_t)T * R * 4);
    if (T <= NVFP4_MMAX) {  // the decode / verify caller; more rows only go through dense_proj below
        eng.dense_ffn_w(mlp, x.ptr(), T, h.ptr(), y.ptr(), xbf16);
        eng.check();
        from_dev(h, dir + "/h.bin");
        from_dev(y, dir + "/y.bin");
    }
    if (T == 1 && !xbf16) {  // the same step captured once and replayed (the reference's CROW_GRAPH path): same bits as the eager launches
        DevBuf hg((size_t)I * 4), yg((size_t)R * 4);
        eng.dense_ffn_w(mlp, x.ptr(), 1, hg.ptr(), yg.ptr());  // eager once more: every Params word exists before the capture
        sync();
        Graph g;
        g.begin();
        eng.dense_ffn_w(mlp, x.ptr(), 1, hg.ptr(), yg.ptr());
        g.end();
        for (int rep = 0; rep < 3; rep++) {
            g.launch();
            g.sync();
        }
        eng.check();
        from_dev(yg, dir + "/y_graph.bin");
    }
    if (!xbf16) {  // dense_proj alone on the same rows, through its own dispatch (t == 1, 2..4, more)
        DevBuf y2((size_t)T * I * 4);
        eng.dense_proj(mlp.gate, T, x.ptr(), y2.ptr());
        eng.check();
        from_dev(y2, dir + "/gate_y.bin");
    }
    return 0;
}

static int head(const std::string& dir) {
    const std::vector<long> m = meta(dir);
    const int V = (int)m.at(0), K = (int)m.at(1);
    const std::vector<uint8_t> gsb = slurp(dir + "/gs.bin");
    Engine eng;
    const Fp4 w = load(dir + "/w.bin", V, K, *(const float*)gsb.data());
    DevBuf x = to_dev(slurp(dir + "/x.bin"));
    DevBuf logits((size_t)V * 4);
    const int tok = eng.lm_head_row(w, x.ptr(), logits.ptr());
    eng.check();
    from_dev(logits, dir + "/logits.bin");
    printf("token=%d\n", tok);
    return 0;
}

static int moe(const std::string& dir) {
    const std::vector<long> m = meta(dir);
    const int E = (int)m.at(0), K = (int)m.at(1), H = (int)m.at(2), I = (int)m.at(3), T = (int)m.at(4);
    const std::vector<uint8_t> gsb = slurp(dir + "/gs.bin");
    const float* gs = (const float*)gsb.data();
    const KernelGeo geo{E, K, H, I};
    Engine eng(&geo);
    const std::vector<uint8_t> gu = slurp(dir + "/gu.bin"), dn = slurp(dir + "/dn.bin");
    const MoeW w = make_moe(load_expert_slabs(gu.data(), gu.size(), E, 2 * I, H, gs[0]), load_expert_slabs(dn.data(), dn.size(), E, H, I, gs[1]));
    DevBuf x = to_dev(slurp(dir + "/x.bin")), logits = to_dev(slurp(dir + "/logits.bin"));
    DevBuf ids((size_t)T * K * 4), wts((size_t)T * K * 4), y((size_t)T * H * 4), h2((size_t)T * K * I * 4), gup((size_t)T * K * 8), dnp((size_t)T * K * 8);
    eng.moe_run(w, T, x.ptr(), logits.ptr(), ids.ptr(), wts.ptr(), y.ptr(), h2.ptr(), gup.ptr(), dnp.ptr());  // y starts as zeros (alloc clears)
    eng.check();
    from_dev(ids, dir + "/ids.bin");
    from_dev(wts, dir + "/wts.bin");
    from_dev(y, dir + "/y.bin");
    return 0;
}

static int moe_grouped(const std::string& dir) {
    const std::vector<long> m = meta(dir);
    const int E = (int)m.at(0), K = (int)m.at(1), H = (int)m.at(2), I = (int)m.at(3), T = (int)m.at(4);
    const std::vector<uint8_t> gsb = slurp(dir + "/gs.bin");
    const float* gs = (const float*)gsb.data();
    const KernelGeo geo{E, K, H, I};
    Engine eng(&geo);
    const std::vector<uint8_t> gu = slurp(dir + "/gu.bin"), dn = slurp(dir + "/dn.bin");
    const MoeW w = make_moe(load_expert_slabs(gu.data(), gu.size(), E, 2 * I, H, gs[0]), load_expert_slabs(dn.data(), dn.size(), E, H, I, gs[1]));
    DevBuf x = to_dev(slurp(dir + "/x.bin")), logits = to_dev(slurp(dir + "/logits.bin"));
    const int combos = T * K, max_tiles = Engine::moe_max_tiles(combos, E);
    DevBuf ids((size_t)combos * 4), wts((size_t)combos * 4), y((size_t)T * H * 4), h2((size_t)combos * I * 4), eo((size_t)combos * H * 4), gup((size_t)combos * 8),
        dnp((size_t)combos * 8), perm((size_t)combos * 4), tiles((size_t)max_tiles * 16), ntl(4);
    eng.moe_run_grouped(w, T, x.ptr(), logits.ptr(), ids.ptr(), wts.ptr(), y.ptr(), h2.ptr(), eo.ptr(), gup.ptr(), dnp.ptr(), perm.ptr(), tiles.ptr(), ntl.ptr());
    eng.check();
    from_dev(ids, dir + "/ids.bin");
    from_dev(wts, dir + "/wts.bin");
    from_dev(y, dir + "/y.bin");
    return 0;
}

static int keeps(const std::string& dir) {  // meta: rows k t; w_bf16.bin (u16), w_f32.bin, x.bin -> y_bf16.bin, y_f32.bin
    const std::vector<long> m = meta(dir);
    const int rows = (int)m.at(0), k = (int)m.at(1), t = (int)m.at(2);
    Engine eng;
    DevBuf wb = to_dev(slurp(dir + "/w_bf16.bin")), wf = to_dev(slurp(dir + "/w_f32.bin")), x = to_dev(slurp(dir + "/x.bin"));
    DevBuf yb((size_t)t * rows * 4), yf((size_t)t * rows * 4);
    eng.bf16_proj(wb.ptr(), rows, k, t, x.ptr(), yb.ptr());
    eng.f32_proj(wf.ptr(), rows, k, t, x.ptr(), yf.ptr());
    eng.check();
    from_dev(yb, dir + "/y_bf16.bin");
    from_dev(yf, dir + "/y_f32.bin");
    return 0;
}

static int gemm(const std::string& dir) {
    const std::vector<long> m = meta(dir);
    const int rows = (int)m.at(0), cols = (int)m.at(1), M = (int)m.at(2);
    const std::vector<uint8_t> gsb = slurp(dir + "/gs.bin");
    Engine eng;
    const Fp4 w = load(dir + "/w.bin", rows, cols, *(const float*)gsb.data());
    DevBuf x = to_dev(slurp(dir + "/x.bin"));
    DevBuf y((size_t)M * rows * 4);
    eng.gemm(w, M, x.ptr(), y.ptr());
    eng.check();
    from_dev(y, dir + "/y.bin");
    return 0;
}

// values.bin (f32) -> blocks.bin, gs.bin through the host layer's encoder; a ragged count must panic with the converter's text
static int quantize(const std::string& dir) {
    const std::vector<uint8_t> raw = slurp(dir + "/values.bin");
    const QuantizedNvfp4 q = quantize_nvfp4((const float*)raw.data(), raw.size() / 4);
    spit(dir + "/blocks.bin", q.blocks.data(), q.blocks.size());
    spit(dir + "/gs.bin", &q.global_scale, sizeof(float));
    try {
        quantize_nvfp4((const float*)raw.data(), 65);
    } catch (const Panic& e) {
        printf("ragged: %s\n", e.what());
    }
    return 0;
}

static int panics() {
    Engine eng;
    try {
        eng.k.f("gemv_nvfp4_nope");
    } catch (const Panic& e) {
        printf("f: %s\n", e.what());
    }
    Fp4 none;
    try {
        eng.proj_m(none, 5, 0, 0);
    } catch (const Panic& e) {
        printf("proj_m: %s\n", e.what());
    }
    return 0;
}

int main(int argc, char** argv) {
    const std::string cmd = argc > 1 ? argv[1] : "";
    try {
        if (cmd == "missing") {
            try {
                launch_dims("gemv_nvfp4_nope", 64, 64);
            } catch (const Panic& e) {
                printf("%s\n", e.what());
            }
            return 0;
        }
        if (cmd == "matrix-checks") {
            const uint8_t b[72] = {0};
            for (int v = 0; v < 2; v++) try {
                    Nvfp4Matrix::make(b, 72, 2, v == 0 ? 96 : 128, 1.0f);
                } catch (const Refused& e) {
                    printf("%s\n", e.what());
                }
            const Nvfp4Matrix ok = Nvfp4Matrix::make(b, 72, 2, 64, 1.0f);
            printf("ok %d %d %zu\n", ok.rows, ok.cols, Nvfp4Matrix::byte_len(17408, 5120));
            return 0;
        }
        if (cmd == "expert-checks") {  // ExpertBlock::new / from_unit refusals and an accepted unit (no GPU needed)
            const size_t gu = Nvfp4Matrix::byte_len(64, 128), dn = Nvfp4Matrix::byte_len(128, 64);
            std::vector<uint8_t> unit(2 * gu + dn, 0);
            const float gsv[3] = {1.0f, 2.0f, 3.0f};
            try {
                ExpertBlock::from_unit(unit.data(), unit.size() - 1, 128, 64, gsv);
            } catch (const Refused& e) {
                printf("%s\n", e.what());
            }
            try {
                ExpertBlock::make(Nvfp4Matrix::make(unit.data(), gu, 64, 128, 1.0f), Nvfp4Matrix::make(unit.data(), gu, 64, 128, 1.0f),
                                  Nvfp4Matrix::make(unit.data(), gu, 64, 128, 1.0f));
            } catch (const Refused& e) {
                printf("%s\n", e.what());
            }
            const ExpertBlock ok = ExpertBlock::from_unit(unit.data(), unit.size(), 128, 64, gsv);
            printf("ok H %d I %d gate %zu up %zu down %zu scales %g %g %g\n", ok.hidden, ok.inter, (size_t)(ok.gate.bytes - unit.data()),
                   (size_t)(ok.up.bytes - unit.data()), (size_t)(ok.down.bytes - unit.data()), ok.gate.global_scale, ok.up.global_scale, ok.down.global_scale);
            return 0;
        }
        if (cmd == "cnq-list" && argc == 3) return cnq_list(argv[2]);
        if (cmd == "cnq-refuse" && argc == 3) {
            try {
                Cnq::open_checked(argv[2]);
                printf("accepted\n");
            } catch (const Refused& e) {
                printf("%s\n", e.what());
            }
            return 0;
        }
        if (cmd == "cnq-dequant" && argc == 4) return cnq_dequant(argv[2], argv[3]);
        if (cmd == "dense" && argc == 3) return dense(argv[2]);
        if (cmd == "head" && argc == 3) return head(argv[2]);
        if (cmd == "moe" && argc == 3) return moe(argv[2]);
        if (cmd == "gemm" && argc == 3) return gemm(argv[2]);
        if (cmd == "moe-grouped" && argc == 3) return moe_grouped(argv[2]);
        if (cmd == "keeps" && argc == 3) return keeps(argv[2]);
        if (cmd == "quantize" && argc == 3) return quantize(argv[2]);
        if (cmd == "panics") return panics();
        fprintf(stderr, "usage: host_parity missing | matrix-checks | cnq-list F | cnq-refuse F | cnq-dequant F DIR | dense DIR | head DIR | moe DIR | gemm DIR | quantize DIR | panics\n");
        return 2;
    } catch (const std::exception& e) {
        fprintf(stderr, "host_parity %s: %s\n", cmd.c_str(), e.what());
        return 1;
    }
}

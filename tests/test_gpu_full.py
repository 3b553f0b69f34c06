"""GPU parity, second file: the device-side ceiling encoder (bit-exact), the router's bookkeeping outputs (bit-exact), launch
dimensions whose row count is read from the device word, an expert unit cut with ``from_unit``, and the benchmark's configs
on WHOLE tensors at the north-star metric (every output row, encoder-made N(0, 0.02^2) weights).

The rule for a whole-tensor comparison (``assert_north_star``): every output is within max relative error 1e-3 of the CPU
path at the 0.1 % floor - or, where one is not, it is an output that cancelled to (almost) nothing and the DEVICE is the
side nearer to an f64 evaluation of the same product; and every output, with no floor, is inside the reference's own
acceptance bound gamma(K/16 + 10) * sum|w x| around that f64 evaluation (engine/src/cpu_nvfp4.rs:491-536).
"""
import json
import os
import struct

import numpy as np
import pytest
import torch

from conftest import GOLDEN
from gpu_common import FLOOR, FLOOR_CHAINED, TOL, quantized_normal, rel_err, rel_l2
from oracle import oracle as orc
from refgen import lcg_bf16_tensors, normal_f32, random_nvfp4

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def eng():
    from crow_nest_amd.engine import Engine
    from crow_nest_amd.kernels import KernelGeo
    return Engine(KernelGeo(experts=256, topk=8, hidden=2048, inter=512))


def _load(w, rows, cols, gs):
    from crow_nest_amd.weights import Nvfp4Matrix, load_fp4
    return load_fp4(Nvfp4Matrix.new(w, rows, cols, gs))


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_north_star(y, ref, w, rows, cols, gs, x, what=""):
    """See the module text.  y, ref: [tokens][rows] (or [rows]); returns (max rel err at the floor, gamma ratio, outputs that
    needed the f64 comparison)."""
    y = np.asarray(y, np.float64).reshape(-1, rows)
    r = np.asarray(ref, np.float64).reshape(-1, rows)
    y64, ab = orc.gemv_f64(w, rows, cols, gs, x)
    y64, ab = y64.reshape(-1, rows), ab.reshape(-1, rows)
    rms = np.sqrt((r * r).mean(axis=1, keepdims=True))
    err = np.abs(y - r) / np.maximum(np.abs(r), FLOOR * np.maximum(rms, 1e-30))
    gam = np.abs(y - y64) / np.maximum(orc.gamma(cols) * ab, np.finfo(np.float64).tiny)
    assert gam.max() <= 1.0, (what, "outside the reference's fp32 bound", float(gam.max()))
    over = err > TOL
    if over.any():
        # only outputs that cancelled: small against their row, and the device no farther from f64 than the CPU path
        assert np.all(np.abs(r[over]) <= 0.02 * np.broadcast_to(rms, r.shape)[over]), (what, "a large output beyond 1e-3")
        assert np.all(np.abs(y[over] - y64[over]) <= np.abs(r[over] - y64[over])), (what, "the device is the farther side from f64")
        assert err.max() <= 2.0 * TOL, (what, float(err.max()))
    return float(err.max()), float(gam.max()), int(over.sum())


# ---------------------------------------------------------------- the encoder (byte-exact)

def _cnq_index():
    raw = open(os.path.join(GOLDEN, "synthetic-v2.cnq"), "rb").read()
    n = struct.unpack("<Q", raw[-8:])[0]
    return raw, json.loads(raw[-8 - n:-8])


def test_device_encoder_reproduces_the_reference_container_byte_for_byte(eng):
    """The six NVFP4 tensors and global scales of the reference's own fixture container, from their LCG source, through
    crow_hip_quantize_nvfp4 (the reference's test does the same with its encoder: converter/src/main.rs:2611-2672)."""
    from crow_nest_amd.weights import quantize_nvfp4
    raw, idx = _cnq_index()
    src = lcg_bf16_tensors()
    seen = 0
    for t in idx["tensors"]:
        if t["dtype"] != "nvfp4":
            continue
        seen += 1
        at = idx["blob_offset"] + t["offset"]
        want = np.frombuffer(raw[at:at + t["len"]], np.uint8)
        blocks, gs = quantize_nvfp4(_dev(src[t["name"]]))
        eng.check()
        assert np.array_equal(blocks.cpu().numpy(), want), t["name"]
        assert gs.cpu().numpy().view(np.uint32)[0] == np.float32(t["global_scale"]).view(np.uint32), t["name"]
    assert seen == 6


def test_device_encoder_equals_the_cpu_encoder_on_hard_inputs(eng):
    """Byte equality with the restated converter encoder on: the benchmark's N(0, 0.02^2) weights; a tensor whose sub-block
    maxima sweep all 127 scale bytes and the subnormal ladder (every power-of-two boundary and its neighbours); a forced
    0x7F sub-block (the tensor's largest raw scale, and one just below the byte before); zeros, signed zeros, values that
    tie exactly on the E2M1 midpoints; an all-zero tensor (global scale 1)."""
    from crow_nest_amd.weights import quantize_nvfp4
    g = np.random.default_rng(5)
    cases = {}
    cases["normal"] = normal_f32(0, 77, 64 * 40000, 0.02)
    # sub-block maxima = 6 * 448 * every representable scale value and its two f32 neighbours, relative to a tensor maximum
    # of 6 * 448 (global scale exactly 1): r = the value itself
    vals = []
    for b in range(0x80):
        v = float(orc.ue4m3(b)) if b < 0x7F else 480.0
        for u in (-1, 0, 1):
            vals.append(np.nextafter(np.float32(v), np.float32(np.inf if u > 0 else -np.inf)) if u else np.float32(v))
    vals = np.array([v for v in vals if 0 < v <= 448.0], np.float32)
    sweep = np.zeros((vals.size + 1, 16), np.float32)
    sweep[:-1, 0] = vals * np.float32(6.0)
    sweep[:-1, 1:] = (g.random((vals.size, 15), dtype=np.float32) * 2 - 1) * sweep[:-1, :1]
    sweep[-1, 3] = np.float32(-6.0 * 448.0)  # the tensor's maximum: byte 0x7E exactly, global scale 1
    pad = (-sweep.shape[0]) % 4
    cases["sweep"] = np.concatenate([sweep, np.zeros((pad, 16), np.float32)]).reshape(-1)
    # ceil rounding makes the largest sub-block land on 0x7F when max / 448 rounds down: search a maximum that does
    forced = normal_f32(1, 78, 64 * 64, 0.02)
    hit = None
    for k in range(4000):
        m = np.float32(0.11) + np.float32(k) * np.float32(1e-5)
        raw = np.float32(m) / np.float32(6.0)
        glob = raw / np.float32(448.0)
        if np.float32(raw / glob) > np.float32(448.0):
            hit = m
            break
    assert hit is not None
    forced[100] = hit
    cases["forced 0x7F"] = forced
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 0.0, -0.0, 6.0, -6.0, 3.0, -0.25, -5.0, 1.0, 0.5], np.float32)
    cases["midpoints"] = np.tile(mids, 8).astype(np.float32)
    cases["zeros"] = np.zeros(128, np.float32)
    tiny = (g.random(64 * 50, dtype=np.float32) * np.float32(1e-3)).astype(np.float32)
    tiny[7] = 100.0  # everything else is far down the subnormal ladder of the scale format
    cases["ladder"] = tiny
    for name, v in cases.items():
        want, gs_want = orc.quantize_ceil(v)
        blocks, gs = quantize_nvfp4(_dev(v))
        eng.check()
        got = blocks.cpu().numpy()
        assert np.array_equal(got, want), (name, int(np.argmax(got != want)))
        assert gs.cpu().numpy().view(np.uint32)[0] == np.float32(gs_want).view(np.uint32), name
    assert 0x7F in orc.quantize_ceil(cases["forced 0x7F"])[0].reshape(-1, 36)[:, :4]
    sc = orc.quantize_ceil(cases["sweep"])[0].reshape(-1, 36)[:, :4].reshape(-1)
    assert len(set(sc.tolist())) >= 126  # every byte of the format but 0x7F (no r beyond 448 in this tensor)


def test_device_encoder_refuses_what_is_not_whole_blocks(eng):
    from crow_nest_amd import lib as L
    v = torch.zeros(96, dtype=torch.float32, device="cuda")
    out = torch.zeros(72, dtype=torch.uint8, device="cuda")
    gs = torch.zeros(1, dtype=torch.float32, device="cuda")
    assert L.lib().crow_hip_quantize_nvfp4(v.data_ptr(), 96, out.data_ptr(), gs.data_ptr()) == -7  # CROW_ERR_SHAPE
    assert L.lib().crow_hip_quantize_nvfp4(0, 64, out.data_ptr(), gs.data_ptr()) == -3
    eng.check()


# ---------------------------------------------------------------- the router's bookkeeping outputs (bit-exact)

@pytest.mark.parametrize("t", [1, 4, 64])
def test_router_bookkeeping_outputs(eng, t):
    """router_top10's warm-up bookkeeping (engine/src/kernels.rs:3170-3183): per-expert selection counts (every routed choice
    counts), the per-token cold mask (bit e = pick e's expert is not in the residency bitmap), and the layer counters
    [selections, cold] - all accumulated onto what the buffers held."""
    from crow_nest_amd.kernels import launch_v
    E, K = 256, 8
    g = np.random.default_rng(100 + t)
    logits = g.standard_normal((t, E)).astype(np.float32)
    if t >= 4:
        logits[1, [200, 9, 77]] = 4.0  # a tie for the top
    bitmap = g.integers(0, 2 ** 32, size=E // 32, dtype=np.uint64).astype(np.uint32)
    sel0 = g.integers(0, 1000, size=E).astype(np.uint64)
    cnt0 = np.array([12345678901, 17], np.uint64)
    ld, bd = _dev(logits), _dev(bitmap.view(np.int32))
    ids = torch.empty((t, K), dtype=torch.int32, device="cuda")
    wts = torch.empty((t, K), dtype=torch.float32, device="cuda")
    cold = torch.full((t,), -1, dtype=torch.int32, device="cuda")
    counters, sel = _dev(cnt0.view(np.int64)), _dev(sel0.view(np.int64))
    launch_v(eng.k.f("router_top10"), t, 1, 1, 64, [ld.data_ptr(), bd.data_ptr(), ids.data_ptr(), wts.data_ptr(), 0, 0, 0,
                                                   cold.data_ptr(), counters.data_ptr(), sel.data_ptr()])
    eng.check()
    ids_ref, _ = orc.router_topk(logits, K)
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    want_sel = sel0.copy()
    np.add.at(want_sel, ids_ref.reshape(-1), 1)
    resident = (bitmap[ids_ref >> 5] >> (ids_ref & 31).astype(np.uint32)) & 1
    want_cold = ((1 - resident.astype(np.uint32)) << np.arange(K, dtype=np.uint32)[None, :]).sum(axis=1).astype(np.uint32)
    assert np.array_equal(sel.cpu().numpy().view(np.uint64), want_sel)
    assert np.array_equal(cold.cpu().numpy().view(np.uint32), want_cold)
    pop = sum(bin(int(c)).count("1") for c in want_cold)
    assert counters.cpu().numpy().view(np.uint64).tolist() == [int(cnt0[0]) + t * K, int(cnt0[1]) + pop]
    # a second launch accumulates again
    launch_v(eng.k.f("router_top10"), t, 1, 1, 64, [ld.data_ptr(), bd.data_ptr(), ids.data_ptr(), wts.data_ptr(), 0, 0, 0,
                                                   cold.data_ptr(), counters.data_ptr(), sel.data_ptr()])
    eng.check()
    assert np.array_equal(sel.cpu().numpy().view(np.uint64), 2 * want_sel - sel0)
    assert counters.cpu().numpy().view(np.uint64).tolist() == [int(cnt0[0]) + 2 * t * K, int(cnt0[1]) + 2 * pop]


# ---------------------------------------------------------------- the row count read from the device word

def test_one_set_of_dimensions_serves_every_row_count(eng):
    """crow_hip_launch_dims with CROW_DIMS_COUNT_FROM_MEMORY (or z = 0 for the verify kernels): the reference's convention
    (a fixed grid, *m_p rewritten per step: kernels_p2.rs:472-497, gen.rs:5455-5466).  Rows hold the same bits as under
    dimensions bound to the count, for every M and T; a captured launch replays correctly after the word has changed."""
    from crow_nest_amd.kernels import COUNT_FROM_MEMORY, Graph, launch_dims, launch_v
    rows, cols = 700, 1024
    w = random_nvfp4(9, rows, cols)
    f = _load(w, rows, cols, 6.0e-4)
    p = eng.p
    x_host = normal_f32(3, 3, 8 * cols).reshape(8, cols)
    bits = orc.f32_to_bf16_bits(x_host)
    x, xb = _dev(x_host), torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16).reshape(8, cols)
    x_wide = orc.bf16_bits_to_f32(bits).reshape(8, cols)  # what the bf16 twin multiplies by
    free = launch_dims("gemv_nvfp4_wm", rows, cols, 0)
    assert free == launch_dims("gemv_nvfp4_wm", rows, cols, COUNT_FROM_MEMORY | 4) and (free[1] >> 20) & 0xF == 0
    m_word = torch.zeros(1, dtype=torch.int32, device="cuda")
    for name, xin in (("gemv_nvfp4_wm", x), ("gemv_nvfp4_wm_bf16", xb)):
        d0 = launch_dims(name, rows, cols, 0)
        for m in (1, 2, 3, 4):
            y_bound = torch.full((4, rows), -7.0, dtype=torch.float32, device="cuda")
            y_free = torch.full((4, rows), -7.0, dtype=torch.float32, device="cuda")
            launch_v(eng.k.f(name), *launch_dims(name, rows, cols, m), [f.w_ptr, xin.data_ptr(), f.gs_ptr, y_bound.data_ptr(), p.i32(cols), p.i32(rows), p.i32(m)])
            m_word.fill_(m)
            launch_v(eng.k.f(name), *d0, [f.w_ptr, xin.data_ptr(), f.gs_ptr, y_free.data_ptr(), p.i32(cols), p.i32(rows), m_word.data_ptr()])
            eng.check()
            assert torch.equal(y_bound.view(torch.int32), y_free.view(torch.int32)), (name, m)
            assert bool((y_free[m:] == -7.0).all()), (name, m)
            err = rel_err(y_free[:m].cpu().numpy(), orc.gemv(w, rows, cols, 6.0e-4, (x_host if name == "gemv_nvfp4_wm" else x_wide)[:m]))
            assert err <= TOL, (name, m, err)
    # token rows: capacity 8, any count up to it
    dcap = launch_dims("gemv_fp4_b", rows, cols, COUNT_FROM_MEMORY | 8)
    for tcount in (1, 5, 8):
        y_bound = torch.full((8, rows), -7.0, dtype=torch.float32, device="cuda")
        y_free = torch.full((8, rows), -7.0, dtype=torch.float32, device="cuda")
        launch_v(eng.k.f("gemv_fp4_b"), *launch_dims("gemv_fp4_b", rows, cols, tcount), [f.w_ptr, x.data_ptr(), f.gs_ptr, y_bound.data_ptr(), p.i32(cols), p.i32(rows), p.i32(tcount)])
        m_word.fill_(tcount)
        launch_v(eng.k.f("gemv_fp4_b"), *dcap, [f.w_ptr, x.data_ptr(), f.gs_ptr, y_free.data_ptr(), p.i32(cols), p.i32(rows), m_word.data_ptr()])
        eng.check()
        assert torch.equal(y_bound.view(torch.int32), y_free.view(torch.int32)), tcount
    # one captured launch, the word rewritten between replays
    y_g = torch.full((4, rows), -7.0, dtype=torch.float32, device="cuda")
    d0 = launch_dims("gemv_nvfp4_wm", rows, cols, 0)
    m_word.fill_(2)
    torch.cuda.synchronize()
    gr = Graph()
    with gr.capture():
        launch_v(eng.k.f("gemv_nvfp4_wm"), *d0, [f.w_ptr, x.data_ptr(), f.gs_ptr, y_g.data_ptr(), p.i32(cols), p.i32(rows), m_word.data_ptr()])
    for m in (2, 4, 1, 3):
        m_word.fill_(m)
        y_g.fill_(-7.0)
        torch.cuda.synchronize()
        gr.launch()
        gr.sync()
        y_e = torch.full((4, rows), -7.0, dtype=torch.float32, device="cuda")
        launch_v(eng.k.f("gemv_nvfp4_wm"), *launch_dims("gemv_nvfp4_wm", rows, cols, m), [f.w_ptr, x.data_ptr(), f.gs_ptr, y_e.data_ptr(), p.i32(cols), p.i32(rows), p.i32(m)])
        eng.check()
        assert torch.equal(y_g.view(torch.int32), y_e.view(torch.int32)), m
    gr.close()
    # kernels that take no count refuse the flag
    from crow_nest_amd.lib import CrowHipError
    with pytest.raises(CrowHipError):
        launch_dims("gemv_nvfp4_w", rows, cols, COUNT_FROM_MEMORY | 1)


# ---------------------------------------------------------------- an expert unit (gate | up | down, three global scales)

def test_an_expert_unit_cut_with_from_unit_runs_its_ffn(eng):
    """ExpertBlock::from_unit (engine/src/cpu_nvfp4.rs:165-178) -> the three matrices on the device -> gate/up + SiLU and
    down, against the CPU path's expert_ffn (cpu_nvfp4.rs:378-427) on the same unit."""
    from crow_nest_amd.weights import ExpertBlock, Nvfp4Matrix, load_expert_block
    hidden, inter = 1024, 384
    gu, dn = Nvfp4Matrix.byte_len(inter, hidden), Nvfp4Matrix.byte_len(hidden, inter)
    unit = np.concatenate([random_nvfp4(1, inter, hidden), random_nvfp4(2, inter, hidden), random_nvfp4(3, hidden, inter)])
    scales = (2.0e-3, 1.5e-3, 1.1e-3)
    e = ExpertBlock.from_unit(unit, hidden, inter, scales)
    mlp = load_expert_block(e)
    x = (normal_f32(4, 4, 2 * hidden) * np.float32(0.05)).reshape(2, hidden)
    for t in (1, 2):
        y = eng.dense_ffn_w(mlp, _dev(x[:t]), t).cpu().numpy()
        eng.check()
        ref = orc.ffn(unit[:gu], scales[0], unit[gu:2 * gu], scales[1], unit[2 * gu:], scales[2], hidden, inter, x[:t])
        assert rel_err(y, ref, FLOOR_CHAINED) <= TOL
        assert rel_l2(y, ref) <= 1e-4


# ---------------------------------------------------------------- whole tensors at the north-star metric

def test_config0_every_row_at_the_north_star_metric(eng):
    rows, cols = 17408, 5120
    w, gs = quantized_normal(0, 0, rows, cols)
    x = normal_f32(0, 1, cols)
    y = eng.dense_proj(_load(w, rows, cols, gs), 1, _dev(x)).cpu().numpy()
    eng.check()
    e, g_, n = assert_north_star(y, orc.gemv(w, rows, cols, gs, x, threads=8), w, rows, cols, gs, x, "config 0")
    print(f"config 0, all {rows} rows: max rel err {e:.3g}, gamma ratio {g_:.3g}, outputs compared through f64: {n}", flush=True)


@pytest.mark.parametrize("m", [1, 2, 4])
def test_config1_down_every_row_at_the_north_star_metric(eng, m):
    """The benchmark's down projection [5120, 17408] on the H the device's own gate/up + SiLU wrote (bf16 X), M = 1, 2, 4:
    all 5120 rows of every token row, one product."""
    from crow_nest_amd.engine import MlpW
    H, I = 5120, 17408
    (wg, gg), (wu, gu), (wd, gd) = quantized_normal(0, 0, I, H), quantized_normal(0, 1, I, H), quantized_normal(0, 2, H, I)
    mlp = MlpW(_load(wg, I, H, gg), _load(wu, I, H, gu), _load(wd, H, I, gd))
    bits = orc.f32_to_bf16_bits(normal_f32(0, 3, 4 * H))
    xb = torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16).reshape(4, H)[:m].contiguous()
    xw = orc.bf16_bits_to_f32(bits).reshape(4, H)[:m]
    h_dev = eng.gate_up(mlp, m, xb)
    y = eng.dense_proj(mlp.down, m, h_dev).cpu().numpy()
    eng.check()
    h = h_dev.cpu().numpy()
    # gate / up + SiLU on all 17408 rows: two products and a SwiGLU, each held to the plain floor through its own product
    g_ref, u_ref = orc.gemv(wg, I, H, gg, xw, threads=8), orc.gemv(wu, I, H, gu, xw, threads=8)
    assert rel_err(h, orc.silu_mul(g_ref, u_ref), FLOOR_CHAINED) <= TOL
    e, g_, n = assert_north_star(y, orc.gemv(wd, H, I, gd, h, threads=8), wd, H, I, gd, h, f"config 1 down M={m}")
    print(f"config 1 down, M = {m}, all {H} rows: max rel err {e:.3g}, gamma ratio {g_:.3g}, outputs compared through f64: {n}", flush=True)


def test_config3_whole_head_on_encoder_made_weights(eng):
    """[151936, 5120] N(0, 0.02^2) through the DEVICE encoder (the bytes are checked against the CPU encoder on a slab), every
    logit against the CPU path, and the greedy token against the argmax of the CPU path's logits - with the margin between
    the two largest logits reported, which is what makes the index comparison meaningful."""
    from crow_nest_amd.weights import load_fp4_quantized, quantize_nvfp4
    rows, cols = 151936, 5120
    blocks_host = np.empty(rows * cols // 64 * 36, np.uint8)
    vals_dev = torch.empty(rows * cols, dtype=torch.float32, device="cuda")
    step = 8192 * cols  # rows per chunk of the generator
    for i, r0 in enumerate(range(0, rows, 8192)):
        n = min(step, rows * cols - r0 * cols)
        vals_dev[r0 * cols:r0 * cols + n] = _dev(normal_f32(0, 1000 + i, n, 0.02))
    blocks, gs_dev = quantize_nvfp4(vals_dev)
    eng.check()
    slab = vals_dev[:4096 * cols].cpu().numpy()
    blocks_host[:] = blocks.cpu().numpy()
    gs = float(gs_dev.cpu().numpy()[0])
    # the same global scale must come out of the CPU encoder when it sees the tensor's maximum: encode a slab that contains it
    want_slab, _ = orc.quantize_ceil(np.concatenate([slab, vals_dev[int(torch.argmax(vals_dev.abs()).item()) // 64 * 64:][:64].cpu().numpy()]))
    assert np.array_equal(blocks_host[:4096 * cols // 64 * 36], want_slab[:4096 * cols // 64 * 36])
    del vals_dev, slab
    f = load_fp4_quantized(blocks, gs_dev, rows, cols)
    x = normal_f32(0, 5, cols)
    logits, idx = eng.lm_head_row(f, _dev(x), fused=True)
    eng.check()
    got = logits.cpu().numpy().reshape(-1)
    ref = orc.gemv(blocks_host, rows, cols, gs, x, threads=8)[0]
    e, g_, n = assert_north_star(got, ref, blocks_host, rows, cols, gs, x, "config 3")
    top2 = np.sort(ref)[-2:]
    print(f"config 3, all {rows} logits: max rel err {e:.3g}, gamma ratio {g_:.3g}, through f64: {n}; top-2 margin {(top2[1] - top2[0]) / abs(top2[1]):.3g}", flush=True)
    assert int(idx.item()) == int(np.argmax(ref)) == orc.argmax_ref(ref)
    logits2, idx2 = eng.lm_head_row(f, _dev(x), fused=False)
    assert int(idx2.item()) == int(idx.item())
    assert np.array_equal(logits2.cpu().numpy().reshape(-1).view(np.uint32), got.view(np.uint32))
    eng.check()


@pytest.mark.parametrize("t", [1, 4])
def test_config2_moe_layer_on_encoder_made_weights(eng, t):
    """256 experts of N(0, 0.02^2) gate|up [1024, 2048] and down [2048, 512] through the device encoder (one global scale per
    tensor, as the container keeps it), router logits N(0, 1), top-8: both launch sequences against the CPU path."""
    from crow_nest_amd.engine import MoeW, expert_table
    from crow_nest_amd.weights import ExpertSlabs, quantize_nvfp4, repack_into, tiled_bytes
    E, H, I, K = 256, 2048, 512, 8
    host = {}
    slabs = {}
    for nm, rows, cols, stream in (("gu", 2 * I, H, 2000), ("dn", H, I, 3000)):
        vals = torch.empty(E * rows * cols, dtype=torch.float32, device="cuda")
        per = 32 * rows * cols
        for i in range(E // 32):
            vals[i * per:(i + 1) * per] = _dev(normal_f32(0, stream + i, per, 0.02))
        blocks, gs = quantize_nvfp4(vals)
        eng.check()
        del vals
        host[nm] = (blocks.cpu().numpy(), float(gs.cpu().numpy()[0]))
        sb, cb = tiled_bytes(rows, cols), rows * cols // 64 * 36
        w = torch.empty(E * sb, dtype=torch.uint8, device="cuda")
        for e_ in range(E):
            repack_into(blocks[e_ * cb:(e_ + 1) * cb], rows, cols, w[e_ * sb:(e_ + 1) * sb])
        slabs[nm] = ExpertSlabs(w, gs, E, rows, cols, sb)
    eng.check()
    moe = MoeW(slabs["gu"], slabs["dn"], expert_table(slabs["gu"], slabs["dn"]))
    x = normal_f32(0, 4000 + t, t * H).reshape(t, H)
    logits = normal_f32(0, 5000 + t, t * E).reshape(t, E)
    ids_ref, w_ref, y_ref = orc.moe_layer(host["gu"][0], host["gu"][1], host["dn"][0], host["dn"][1], E, H, I, x, logits, K, threads=8)
    for fused in ("route", True, False):
        ids, wts, y = eng.moe_run(moe, _dev(x), _dev(logits), fused=fused)
        eng.check()
        assert np.array_equal(ids.cpu().numpy(), ids_ref), fused
        assert np.allclose(wts.cpu().numpy(), w_ref, rtol=2e-6, atol=0), fused
        assert rel_err(y.cpu().numpy(), y_ref, FLOOR_CHAINED) <= TOL, fused
        assert rel_l2(y.cpu().numpy(), y_ref) <= 1e-4, fused

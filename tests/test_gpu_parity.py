"""GPU parity: the HIP path (through the C ABI, via the host mirror) against the CPU oracle.

Bars: dequantised weights bit-exact; integer / index results bit-exact; GEMV outputs within
max relative error 1e-3 of the CPU path (TOL; the denominator floors at 0.1 % of the row's rms so that
an output that cancels to ~0 does not divide by nothing - see gpu_common.rel_err), and additionally
inside the reference's own fp32 bound gamma(K/16 + 10) * sum|w x| against an f64 evaluation
(gamma_ratio; on sampled rows where the tensor is large).
"""
import numpy as np
import pytest
import torch

from gpu_common import FLOOR_CHAINED, TOL, floor_of, gamma_ratio, gamma_rows, quantized_normal, rel_err, rel_l2
from oracle import oracle as orc
from refgen import SplitMix64, normal_f32, random_nvfp4, scale_mix, synth_nvfp4

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


def _bf16_dev(a_f32):
    """RNE to bf16 on the host (the oracle's rounding), bits shipped to the device."""
    bits = orc.f32_to_bf16_bits(a_f32)
    return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16), orc.bf16_bits_to_f32(bits)


# ---------------------------------------------------------------- layout + dequant (bit-exact)

@pytest.mark.parametrize("rows,cols", [(64, 256), (37, 256), (1, 64), (65, 320), (128, 64), (200, 5120), (16, 2048)])
def test_repack_round_trip_and_dequant_bits(eng, rows, cols):
    from crow_nest_amd.weights import dequant, unpack
    print(f"case rows={rows} cols={cols}", flush=True)
    w = random_nvfp4(rows * 1000 + cols, rows, cols, scale_lo=0, scale_hi=0x7F, p7f=1 / 32)
    gs = 1.7e-3
    f = _load(w, rows, cols, gs)
    back = unpack(f)
    canon = w.copy().reshape(-1, 36)
    canon[:, :4][canon[:, :4] == 0x7F] = 0x7E
    assert np.array_equal(back, canon.reshape(-1))  # exact inverse up to the scale rule
    got = dequant(f).cpu().numpy().reshape(-1)
    want = orc.dequant(w, gs)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    eng.check()


def test_dequant_every_scale_byte_and_the_refused_one(eng):
    from crow_nest_amd.lib import CrowHipError
    from crow_nest_amd.weights import dequant
    rows, cols = 256, 64
    blocks = np.zeros((rows, 36), np.uint8)
    g = np.random.default_rng(1)
    blocks[:, 4:] = g.integers(0, 256, size=(rows, 32), dtype=np.uint8)
    for r in range(rows):
        blocks[r, :4] = [r, (r + 64) % 256, (r + 128) % 256, (r + 192) % 256]
    ok = blocks.copy()
    ok[:, :4][ok[:, :4] == 0xFF] = 0x7F
    gs = 9.3e-5
    got = dequant(_load(ok.reshape(-1), rows, cols, gs)).cpu().numpy().reshape(-1)
    want = orc.dequant(ok.reshape(-1), gs)  # bit 7 ignored, 0x7F -> 448
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    with pytest.raises(CrowHipError) as ei:  # 0xFF reads 480 in the reference; the tiled layout cannot hold it
        _load(blocks.reshape(-1), rows, cols, gs)
    assert ei.value.code == -6
    eng.check()


def test_dequant_fp4_flat_is_the_raw_container_decode(eng):
    from crow_nest_amd.kernels import launch_v
    w = random_nvfp4(5, 64, 512, scale_lo=0, scale_hi=0x100, p7f=1 / 16)
    gs = torch.tensor([2.3e-4], dtype=torch.float32, device="cuda")
    n = 64 * 512
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    wd = _dev(w)
    launch_v(eng.k.f("dequant_fp4_flat"), (n + 255) // 256, 1, 1, 256, [wd.data_ptr(), gs.data_ptr(), out.data_ptr(), eng.p.i32(n)])
    want = orc.dequant(w, 2.3e-4, rule=False)  # 0x7F reads 480 here, as in the reference kernel
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


# ---------------------------------------------------------------- dense GEMV

SHAPES = [(37, 256), (16, 2048), (9, 4096), (41, 1024), (64, 64), (130, 320), (1024, 5120), (512, 17408), (2048, 512), (100, 2560)]


@pytest.mark.parametrize("rows,cols", SHAPES)
def test_gemv_w_against_the_cpu_path(eng, rows, cols):
    print(f"case rows={rows} cols={cols}", flush=True)
    rng = SplitMix64(173 + rows)
    w = synth_nvfp4(rng, rows, cols, scale_mix) if rows * cols <= 1 << 18 else random_nvfp4(rows, rows, cols)
    gs = 1.7e-3
    x = rng.f(cols, 2.0)
    ref = orc.gemv(w, rows, cols, gs, x)[0]
    f = _load(w, rows, cols, gs)
    y = eng.dense_proj(f, 1, _dev(x)).cpu().numpy()[0]
    eng.check()
    assert rel_err(y, ref) <= TOL
    assert gamma_ratio(y, w, rows, cols, gs, x) <= 1.0


@pytest.mark.parametrize("s,wv", [(1, 1), (1, 4), (1, 5), (3, 2), (5, 1), (20, 1), (2, 10), (1, 16)])
def test_gemv_is_correct_for_every_split(eng, s, wv):
    """Any (slices, waves) split gives an answer inside the bound; the same split gives the same bits.  (1, 1) and (1, 4) make
    a wave walk more groups than it holds at once: the loop over register loads."""
    rows, cols = 300, 5120
    w = random_nvfp4(77, rows, cols)
    gs = 4.0e-4
    x = normal_f32(1, 5, cols)
    ref = orc.gemv(w, rows, cols, gs, x)[0]
    from crow_nest_amd.kernels import launch_dims, launch_v
    f = _load(w, rows, cols, gs)
    xd, p = _dev(x), eng.p
    dims = launch_dims("gemv_nvfp4_w", rows, cols, 1, split=(s, wv))
    assert dims[1] >> 24 == s and dims[3] == 64 * wv and dims[1] & 0xFFFFF == cols // 64
    ys = []
    for _ in range(2):
        y = torch.empty((1, rows), dtype=torch.float32, device="cuda")
        launch_v(eng.k.f("gemv_nvfp4_w"), *dims, [f.w_ptr, xd.data_ptr(), f.gs_ptr, y.data_ptr(), p.i32(cols), p.i32(rows)])
        ys.append(y.cpu().numpy()[0])
    y1, y2 = ys
    eng.check()
    assert np.array_equal(y1.view(np.uint32), y2.view(np.uint32))
    assert rel_err(y1, ref) <= TOL and gamma_ratio(y1, w, rows, cols, gs, x) <= 1.0


def test_ragged_shapes_drawn_at_random(eng):
    """Forty shapes drawn with a fixed seed - any row count (partial last row tile), any whole number of 64-value blocks per
    row (partial last panel), 1..4 activation rows, f32 or bf16 activations - through dense_proj / proj_m and the fused
    gate/up kernels, each against the CPU path."""
    from crow_nest_amd.engine import MlpW
    g = np.random.default_rng(20240611)
    for case in range(40):
        rows = int(g.integers(1, 260))
        cols = 64 * int(g.integers(1, 41))
        m = int(g.integers(1, 5))
        bf16 = bool(g.integers(0, 2))
        print(f"case {case}: rows={rows} cols={cols} m={m} bf16={bf16}", flush=True)
        w, w2 = random_nvfp4(1000 + case, rows, cols), random_nvfp4(2000 + case, rows, cols)
        gs, gs2 = 7.0e-4, 1.1e-3
        f, f2 = _load(w, rows, cols, gs), _load(w2, rows, cols, gs2)
        x = normal_f32(8, case, m * cols).reshape(m, cols)
        if bf16:
            xb, xw = _bf16_dev(x)
            xd, xo = xb.reshape(m, cols).contiguous(), xw.reshape(m, cols)
        else:
            xd, xo = _dev(x), x
        ref = orc.gemv(w, rows, cols, gs, xo)
        y = (eng.proj_m(f, m, xd) if (bf16 or m > 1) else eng.dense_proj(f, 1, xd)).cpu().numpy()
        assert rel_err(y, ref) <= TOL, case
        assert gamma_ratio(y, w, rows, cols, gs, xo) <= 1.0, case
        h = eng.gate_up(MlpW(f, f2, f), m, xd).cpu().numpy()
        assert rel_err(h, orc.silu_mul(ref, orc.gemv(w2, rows, cols, gs2, xo))) <= TOL, case
    eng.check()


def test_split_launches_back_to_back_with_changing_inputs(eng):
    """A small cross-block split launched 24 times in a row without a host wait, every launch on another x: the partial
    sums a block reads are the ones this launch's blocks wrote, never an earlier launch's (the launches are small enough
    for all of their lines to stay in the caches between them)."""
    rows, cols, n = 128, 4096, 24
    w = random_nvfp4(91, rows, cols)
    gs = 6.0e-4
    f = _load(w, rows, cols, gs)
    from crow_nest_amd.kernels import launch_dims, launch_v
    xs = normal_f32(6, 1, n * cols).reshape(n, cols) * np.linspace(0.25, 4.0, n, dtype=np.float32)[:, None]
    xd = _dev(xs)
    p = eng.p
    for s, wv in ((4, 4), (16, 1), (2, 8)):
        dims = launch_dims("gemv_nvfp4_w", rows, cols, 1, split=(s, wv))
        assert dims[1] >> 24 == s
        y = torch.empty((n, rows), dtype=torch.float32, device="cuda")
        for i in range(n):
            launch_v(eng.k.f("gemv_nvfp4_w"), *dims, [f.w_ptr, xd[i].data_ptr(), f.gs_ptr, y[i].data_ptr(), p.i32(cols), p.i32(rows)])
        eng.check()
        got = y.cpu().numpy()
        ref = orc.gemv(w, rows, cols, gs, xs)
        for i in range(n):
            assert rel_err(got[i], ref[i]) <= TOL, (s, wv, i)


def test_five_thousand_hand_overs_in_a_row_give_the_same_bits(eng):
    """The cross-block hand-over under sustained load: 5,000 launches back to back of the split GEMV at the benchmark's down
    projection size (5 column slices per strip through the workspace) and as many of the K-split 16-token GEMM at full size,
    rotating over 8 inputs; every result is compared bit for bit with the first result for its input (on the device, after
    every round of 8), and the first results with the CPU path."""
    from crow_nest_amd.kernels import launch_dims, launch_v
    p = eng.p
    rounds = 625
    # --- the split GEMV [5120, 17408]
    rows, cols = 5120, 17408
    w = random_nvfp4(501, rows, cols)
    gs = 2.0e-4
    f = _load(w, rows, cols, gs)
    xs = np.stack([normal_f32(502, i, cols) for i in range(8)])
    xd = _dev(xs)
    dims = launch_dims("gemv_nvfp4_w", rows, cols)
    assert dims[1] >> 24 > 1
    y = torch.empty((8, rows), dtype=torch.float32, device="cuda")
    first = None
    for r in range(rounds):
        for i in range(8):
            launch_v(eng.k.f("gemv_nvfp4_w"), *dims, [f.w_ptr, xd[i].data_ptr(), f.gs_ptr, y[i].data_ptr(), p.i32(cols), p.i32(rows)])
        if first is None:
            first = y.clone()
        else:
            assert torch.equal(y.view(torch.int32), first.view(torch.int32)), f"GEMV round {r}"
        y.fill_(-1.0)
    eng.check()
    got = first.cpu().numpy()
    for i in (0, 7):
        assert gamma_rows(got[i][:256], w, 0, 256, cols, gs, xs[i]) <= 1.0
    # --- the K-split GEMM for 16 tokens on [17408, 5120]
    rows, cols, m = 17408, 5120, 16
    w = random_nvfp4(503, rows, cols)
    f = _load(w, rows, cols, gs)
    xb = [_bf16_dev(normal_f32(504, i, m * cols).reshape(m, cols)) for i in range(8)]
    dims = launch_dims("gemm_nvfp4_bf16_m16", rows, cols, m)
    assert dims[2] > 1  # the panels are dealt over several blocks per row tile
    y = torch.empty((8, m, rows), dtype=torch.float32, device="cuda")
    first = None
    for r in range(rounds):
        for i in range(8):
            launch_v(eng.k.f("gemm_nvfp4_bf16_m16"), *dims, [f.w_ptr, xb[i][0].data_ptr(), f.gs_ptr, y[i].data_ptr(), p.i32(cols), p.i32(rows), p.i32(m)])
        if first is None:
            first = y.clone()
        else:
            assert torch.equal(y.view(torch.int32), first.view(torch.int32)), f"GEMM round {r}"
        y.fill_(-1.0)
    eng.check()
    got = first.cpu().numpy()
    assert gamma_rows(got[3][:, :128], w, 0, 128, cols, gs, xb[3][1]) <= 1.0


@pytest.mark.parametrize("name", ["gemv_nvfp4_w_valu1", "gemv_nvfp4_w_valu2", "gemv_nvfp4_w_valu4"])
def test_the_measurement_only_gemv_without_matrix_instructions(eng, name):
    """The A/B kernels (container layout, f32 multiply-adds): same product, within the same bounds."""
    from crow_nest_amd.kernels import launch_dims, launch_v
    p = eng.p
    for rows, cols in [(37, 256), (130, 320), (1000, 5120), (64, 17408)]:
        w = random_nvfp4(700 + rows, rows, cols, scale_lo=0, scale_hi=0x100, p7f=1 / 16)
        w = w.copy().reshape(-1, 36)
        w[:, :4][w[:, :4] == 0xFF] = 0x7F  # (the tiled path refuses 0xFF; keep the comparison on common ground)
        w = w.reshape(-1)
        gs = 7.0e-4
        x = normal_f32(701, rows, cols)
        wd, xd = _dev(w), _dev(x)
        gsd = torch.tensor([gs], dtype=torch.float32, device="cuda")
        y = torch.full((rows,), -7.0, dtype=torch.float32, device="cuda")
        launch_v(eng.k.f(name), *launch_dims(name, rows, cols), [wd.data_ptr(), xd.data_ptr(), gsd.data_ptr(), y.data_ptr(), p.i32(cols), p.i32(rows)])
        eng.check()
        got = y.cpu().numpy()
        assert rel_err(got, orc.gemv(w, rows, cols, gs, x)[0]) <= TOL, (rows, cols)
        assert gamma_ratio(got, w, rows, cols, gs, x) <= 1.0, (rows, cols)


def test_verify_rows_are_bit_identical_to_one_row_decode(eng):
    """kernels_p2.rs:391-396: row m of an M-row launch == a one-row launch on x row m."""
    rows, cols = 700, 5120
    w = random_nvfp4(3, rows, cols)
    gs = 3.1e-4
    f = _load(w, rows, cols, gs)
    x = normal_f32(2, 9, 4 * cols).reshape(4, cols)
    one = [eng.dense_proj(f, 1, _dev(x[m])).cpu().numpy()[0] for m in range(4)]
    for m in (1, 2, 3, 4):
        ym = eng.proj_m(f, m, _dev(x[:m])).cpu().numpy()
        for j in range(m):
            assert np.array_equal(ym[j].view(np.uint32), one[j].view(np.uint32)), (m, j)
        assert rel_err(ym, orc.gemv(w, rows, cols, gs, x[:m])) <= TOL
        assert gamma_ratio(ym, w, rows, cols, gs, x[:m]) <= 1.0
    eng.check()


@pytest.mark.parametrize("t", [1, 2, 4])
def test_fused_gate_up_silu_and_down(eng, t):
    from crow_nest_amd.engine import MlpW
    H, I = 1024, 2816
    wg, wu, wd = random_nvfp4(11, I, H), random_nvfp4(12, I, H), random_nvfp4(13, H, I)
    gs = (2.0e-3, 1.5e-3, 1.1e-3)
    mlp = MlpW(_load(wg, I, H, gs[0]), _load(wu, I, H, gs[1]), _load(wd, H, I, gs[2]))
    x = normal_f32(3, t, t * H).reshape(t, H) * np.float32(0.05)
    # f32 activations (the reference's dtype)
    h = eng.gate_up(mlp, t, _dev(x)).cpu().numpy()
    g_ref, u_ref = orc.gemv(wg, I, H, gs[0], x), orc.gemv(wu, I, H, gs[1], x)
    h_ref = orc.silu_mul(g_ref, u_ref)
    assert rel_err(h, h_ref) <= TOL
    y = eng.dense_ffn_w(mlp, _dev(x), t).cpu().numpy()
    y_ref = orc.ffn(wg, gs[0], wu, gs[1], wd, gs[2], H, I, x)
    assert rel_err(y, y_ref, FLOOR_CHAINED) <= TOL  # two products in a row: see gpu_common.FLOOR_CHAINED
    # each product on its own, at the plain floor and inside the bound of the reference's own gate: down on the device's own h,
    # gate alone through proj_m
    yd = eng.dense_proj(mlp.down, t, _dev(h)).cpu().numpy()
    assert np.array_equal(yd.view(np.uint32), y.view(np.uint32))
    assert rel_err(yd, orc.gemv(wd, H, I, gs[2], h)) <= TOL
    assert gamma_ratio(yd, wd, H, I, gs[2], h) <= 1.0
    assert gamma_ratio(eng.proj_m(mlp.gate, t, _dev(x)).cpu().numpy(), wg, I, H, gs[0], x) <= 1.0
    # bf16 activations (benchmark config 1: bf16 X): the oracle gets the exactly widened values
    xb, xw = _bf16_dev(x)
    hb = eng.gate_up(mlp, t, xb.reshape(t, H).contiguous()).cpu().numpy()
    hb_ref = orc.silu_mul(orc.gemv(wg, I, H, gs[0], xw), orc.gemv(wu, I, H, gs[1], xw))
    assert rel_err(hb, hb_ref) <= TOL
    eng.check()


def test_batched_token_rows(eng):
    rows, cols, t = 192, 1024, 7
    w = random_nvfp4(21, rows, cols)
    gs = 8.0e-4
    f = _load(w, rows, cols, gs)
    x = normal_f32(4, 1, t * cols).reshape(t, cols)
    y = eng.dense_proj(f, t, _dev(x)).cpu().numpy()
    assert rel_err(y, orc.gemv(w, rows, cols, gs, x)) <= TOL
    eng.check()


def test_record_kernel_entry_points_by_their_own_names(eng):
    """gemv_fp4 (kernels.rs:118-151), gemv_fp4_b1k (:1302-1337), gemv_fp4_bs (:1022-1058, its own y stride word) and the
    one-row bf16 twin gemv_nvfp4_w_bf16 (kernels_p2.rs:355-368), each launched through the C ABI under its own name on a
    ragged shape, against the CPU path and inside its f32 bound."""
    from crow_nest_amd.kernels import launch_dims, launch_v
    rows, cols = 203, 1984  # a partial last strip, a partial last group
    w = random_nvfp4(808, rows, cols)
    gs = 9.0e-4
    f = _load(w, rows, cols, gs)
    p = eng.p
    x = normal_f32(9, 1, 5 * cols).reshape(5, cols)
    xd = _dev(x)
    ref = orc.gemv(w, rows, cols, gs, x)
    # gemv_fp4: one row
    y = torch.full((rows,), 7.0, dtype=torch.float32, device="cuda")
    launch_v(eng.k.f("gemv_fp4"), *launch_dims("gemv_fp4", rows, cols), [f.w_ptr, xd[2].data_ptr(), f.gs_ptr, y.data_ptr(), p.i32(cols), p.i32(rows)])
    eng.check()
    assert rel_err(y.cpu().numpy(), ref[2]) <= TOL and gamma_ratio(y.cpu().numpy(), w, rows, cols, gs, x[2]) <= 1.0
    # gemv_nvfp4_w_bf16: one bf16 row
    xb, xw = _bf16_dev(x[3])
    y = torch.full((rows,), 7.0, dtype=torch.float32, device="cuda")
    launch_v(eng.k.f("gemv_nvfp4_w_bf16"), *launch_dims("gemv_nvfp4_w_bf16", rows, cols), [f.w_ptr, xb.data_ptr(), f.gs_ptr, y.data_ptr(), p.i32(cols), p.i32(rows)])
    eng.check()
    assert rel_err(y.cpu().numpy(), orc.gemv(w, rows, cols, gs, xw)[0]) <= TOL and gamma_ratio(y.cpu().numpy(), w, rows, cols, gs, xw) <= 1.0
    # ... and it is the M = 1 case of the verify twin, bit for bit
    y1 = eng.proj_m(f, 1, xb.reshape(1, cols)).cpu().numpy()[0]
    assert np.array_equal(y1.view(np.uint32), y.cpu().numpy().view(np.uint32))
    # gemv_fp4_b1k: five token rows (a full group of four and a last group of one)
    yb = torch.full((5, rows), 7.0, dtype=torch.float32, device="cuda")
    launch_v(eng.k.f("gemv_fp4_b1k"), *launch_dims("gemv_fp4_b1k", rows, cols, 5), [f.w_ptr, xd.data_ptr(), f.gs_ptr, yb.data_ptr(), p.i32(cols), p.i32(rows), p.i32(5)])
    eng.check()
    assert rel_err(yb.cpu().numpy(), ref) <= TOL and gamma_ratio(yb.cpu().numpy(), w, rows, cols, gs, x) <= 1.0
    # gemv_fp4_bs: seven ... here five rows into a wider buffer; the gap columns stay untouched
    stride = rows + 37
    ys = torch.full((5, stride), 7.0, dtype=torch.float32, device="cuda")
    launch_v(eng.k.f("gemv_fp4_bs"), *launch_dims("gemv_fp4_bs", rows, cols, 5),
             [f.w_ptr, xd.data_ptr(), f.gs_ptr, ys.data_ptr(), p.i32(cols), p.i32(stride), p.i32(rows), p.i32(5)])
    eng.check()
    got = ys.cpu().numpy()
    assert np.array_equal(got[:, :rows].view(np.uint32), yb.cpu().numpy().view(np.uint32))  # the same bodies: the same bits
    assert bool((got[:, rows:] == 7.0).all())
    # a stride shorter than a row is refused, nothing written
    from crow_nest_amd.lib import CrowHipError
    ys.fill_(7.0)
    launch_v(eng.k.f("gemv_fp4_bs"), *launch_dims("gemv_fp4_bs", rows, cols, 5),
             [f.w_ptr, xd.data_ptr(), f.gs_ptr, ys.data_ptr(), p.i32(cols), p.i32(rows - 1), p.i32(rows), p.i32(5)])
    with pytest.raises(CrowHipError) as ei:
        eng.check()
    assert ei.value.code == -7 and bool((ys == 7.0).all())
    # dims made for one token count, the word behind t_p saying another: refused
    launch_v(eng.k.f("gemv_fp4_b"), *launch_dims("gemv_fp4_b", rows, cols, 5), [f.w_ptr, xd.data_ptr(), f.gs_ptr, ys.data_ptr(), p.i32(cols), p.i32(rows), p.i32(4)])
    with pytest.raises(CrowHipError) as ei:
        eng.check()
    assert ei.value.code == -7 and bool((ys == 7.0).all())
    eng.check()


# ---------------------------------------------------------------- head

def test_lm_head_logits_and_greedy_token(eng):
    rows, cols = 4096 + 64 * 3, 1024
    w, gs = quantized_normal(0, 31, rows, cols)
    f = _load(w, rows, cols, gs)
    x = normal_f32(0, 32, cols)
    ref = orc.gemv(w, rows, cols, gs, x)[0]
    for fused in (True, False):
        logits, idx = eng.lm_head_row(f, _dev(x), fused=fused)
        got = logits.cpu().numpy()
        assert rel_err(got, ref) <= TOL
        assert int(idx.item()) == orc.argmax_ref(got)  # the index is exact on the logits the device wrote
    assert int(idx.item()) == int(np.argmax(ref))
    eng.check()


def test_argmax_tie_rule(eng):
    for n, hot in [(4096, [1030, 7, 2055]), (151936, [150000, 1023 + 1024 * 3, 1023]), (5, [4, 2]), (2048, [1, 1536, 512]),
                   (151936, [3, 5, 6, 9, 10, 12, 100000]), (3000, [])]:
        l = np.zeros(n, np.float32) if hot else np.full(n, -3.2e38, np.float32)
        for i in hot:
            l[i] = 5.0
        got = int(eng.argmax(_dev(l)).item())
        assert got == orc.argmax_ref(l), (n, hot)
    g = np.random.default_rng(8)
    l = g.standard_normal(151936).astype(np.float32)
    assert int(eng.argmax(_dev(l)).item()) == int(np.argmax(l))


def test_fused_head_tie_rule(eng):
    """Equal logits in different row tiles: the fused head must pick by the reference's tree order too."""
    rows, cols = 2048 + 128, 64
    blocks = np.zeros((rows, 36), np.uint8)
    blocks[:, 0] = 0x38  # scale 1.0
    for r in (1030, 7, 2055):  # value 2 (code 4) at column 0
        blocks[r, 4] = 0x04
    f = _load(blocks.reshape(-1), rows, cols, 1.0)
    x = np.ones(cols, np.float32)
    logits, idx = eng.lm_head_row(f, _dev(x), fused=True)
    l = logits.cpu().numpy()
    assert l[7] == 2.0 and l[1030] == 2.0 and l[0] == 0.0
    assert int(idx.item()) == orc.argmax_ref(l) == 1030
    eng.check()


# ---------------------------------------------------------------- routed experts

def test_router_small_kernels(eng):
    g = np.random.default_rng(12)
    logits = g.standard_normal((5, 256)).astype(np.float32)
    logits[3, [9, 200, 77]] = 4.0  # three-way tie for the top: lowest ids first
    ids, wts, _, _ = eng.router(_dev(logits))
    ids_ref, w_ref = orc.router_topk(logits, 8)
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    assert np.allclose(wts.cpu().numpy(), w_ref, rtol=2e-6, atol=0)  # device expf vs libm expf: last-ulp
    assert ids_ref[3, :3].tolist() == [9, 77, 200]
    # SwiGLU per combo and the weighted combine: same f32 operations as the oracle -> bit-exact
    from crow_nest_amd.kernels import launch_v
    h1 = g.standard_normal((40, 1024)).astype(np.float32)
    h2 = torch.empty((40, 512), dtype=torch.float32, device="cuda")
    h1d = _dev(h1)
    launch_v(eng.k.f("silu_mul_combo"), (40 * 512 + 255) // 256, 1, 1, 256, [h1d.data_ptr(), h2.data_ptr(), eng.p.i32(40 * 512)])
    assert np.allclose(h2.cpu().numpy(), orc.silu_mul_combo(h1, 512), rtol=1e-6, atol=1e-30)
    eo = g.standard_normal((5 * 8, 2048)).astype(np.float32)
    rw = g.random((5, 8)).astype(np.float32)
    y0 = g.standard_normal((5, 2048)).astype(np.float32)
    y = _dev(y0.copy())
    eod, rwd = _dev(eo), _dev(rw)
    launch_v(eng.k.f("acc_combo"), 2048 // 256, 5, 1, 256, [eod.data_ptr(), rwd.data_ptr(), y.data_ptr()])
    want = orc.acc_combo(eo, rw, 5, 8, 2048, y0)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
    eng.check()


@pytest.mark.parametrize("experts,topk", [(64, 4), (128, 8), (512, 10), (1024, 16)])
def test_router_other_geometries_and_ties(eng, experts, topk):
    """Expert counts from one to sixteen per lane; equal logits in several lanes and inside one lane (ties go to the
    lowest expert id); a whole row of equal logits."""
    from crow_nest_amd.kernels import KernelGeo, launch_v, set_geo
    print(f"case experts={experts} topk={topk}", flush=True)
    g = np.random.default_rng(experts)
    logits = g.standard_normal((6, experts)).astype(np.float32)
    logits[1, [5, 5 + 64 % experts, experts - 1, 17]] = 3.5  # same lane (where experts > 64) and other lanes
    logits[2, :] = 0.25                                       # everything ties: ids 0 .. topk-1
    logits[3, experts // 2:] = logits[3, : experts // 2]     # every value twice, 'experts / 2' apart
    logits[4, [experts - 1, experts - 2]] = 9.0
    try:
        set_geo(KernelGeo(experts=experts, topk=topk, hidden=2048, inter=512))
        ld = _dev(logits)
        ids = torch.empty((6, topk), dtype=torch.int32, device="cuda")
        wts = torch.empty((6, topk), dtype=torch.float32, device="cuda")
        launch_v(eng.k.f("router_top10"), 6, 1, 1, 64, [ld.data_ptr(), 0, ids.data_ptr(), wts.data_ptr(), 0, 0, 0, 0, 0, 0])
        eng.check()
    finally:
        set_geo(eng.geo)
    ids_ref, w_ref = orc.router_topk(logits, topk)
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    assert np.allclose(wts.cpu().numpy(), w_ref, rtol=2e-6, atol=0)
    assert ids_ref[2].tolist() == list(range(topk))


def test_two_geometries_interleaved_without_a_wait(eng):
    """The geometry rides on every launch by value: routing launches of two geometries queued alternately on one stream,
    with nothing waited for in between, each use their own."""
    from crow_nest_amd.kernels import KernelGeo, launch_v, set_geo
    geos = [KernelGeo(experts=64, topk=4, hidden=2048, inter=512), KernelGeo(experts=512, topk=10, hidden=2048, inter=512)]
    g = np.random.default_rng(99)
    logits = [g.standard_normal((5, ge.experts)).astype(np.float32) for ge in geos for _ in range(3)]
    devs = [_dev(l) for l in logits]
    outs = []
    try:
        order = [0, 3, 1, 4, 2, 5]  # the data is A, A, A, B, B, B; launched A, B, A, B, A, B
        for i in order:
            ge = geos[i // 3]
            set_geo(ge)
            ids = torch.empty((5, ge.topk), dtype=torch.int32, device="cuda")
            wts = torch.empty((5, ge.topk), dtype=torch.float32, device="cuda")
            launch_v(eng.k.f("router_top10"), 5, 1, 1, 64, [devs[i].data_ptr(), 0, ids.data_ptr(), wts.data_ptr(), 0, 0, 0, 0, 0, 0])
            outs.append((i, ids, wts))
        eng.check()
    finally:
        set_geo(eng.geo)
    for i, ids, wts in outs:
        ids_ref, w_ref = orc.router_topk(logits[i], geos[i // 3].topk)
        assert np.array_equal(ids.cpu().numpy(), ids_ref), i
        assert np.allclose(wts.cpu().numpy(), w_ref, rtol=2e-6, atol=0), i


@pytest.mark.parametrize("t", [1, 4])
def test_moe_layer_both_launch_sequences(eng, t):
    from crow_nest_amd.engine import MoeW, expert_table
    from crow_nest_amd.weights import load_expert_slabs
    E, H, I, K = 256, 2048, 512, 8
    gu = random_nvfp4(41, E * 2 * I, H, scale_lo=0x30, scale_hi=0x48, p7f=0)
    dn = random_nvfp4(42, E * H, I, scale_lo=0x30, scale_hi=0x48, p7f=0)
    gs_gu, gs_dn = 2.0e-3, 3.0e-3
    s_gu, s_dn = load_expert_slabs(gu, E, 2 * I, H, gs_gu), load_expert_slabs(dn, E, H, I, gs_dn)
    moe = MoeW(s_gu, s_dn, expert_table(s_gu, s_dn))
    x = (normal_f32(5, t, t * H) * np.float32(0.1)).reshape(t, H)
    logits = normal_f32(6, t, t * E).reshape(t, E)
    ids_ref, w_ref, y_ref = orc.moe_layer(gu, gs_gu, dn, gs_dn, E, H, I, x, logits, K, threads=8)
    for fused in (False, True, "route"):
        print(f"case moe t={t} fused={fused}", flush=True)
        ids, wts, y = eng.moe_run(moe, _dev(x), _dev(logits), fused=fused)
        eng.check()
        assert np.array_equal(ids.cpu().numpy(), ids_ref)
        assert np.allclose(wts.cpu().numpy(), w_ref, rtol=2e-6, atol=0)
        assert rel_err(y.cpu().numpy(), y_ref, FLOOR_CHAINED) <= TOL, fused  # products in a row: gpu_common.FLOOR_CHAINED
    eng.check()


def test_routed_expert_products_inside_the_bound(eng):
    """The two products of a routed layer on their own, per combo: gemv_fp4_ptrb on the gate|up slabs and on the down slabs
    (kernels.rs:195-233), and the fused moe_gate_up_silu, against the CPU path on the same expert's container bytes, at the
    plain floor and inside the f32 bound."""
    from crow_nest_amd.engine import expert_table
    from crow_nest_amd.kernels import launch_dims, launch_v
    from crow_nest_amd.weights import load_expert_slabs
    E, H, I, K = 256, 2048, 512, 8
    gu = random_nvfp4(41, E * 2 * I, H, scale_lo=0x30, scale_hi=0x48, p7f=0)
    dn = random_nvfp4(42, E * H, I, scale_lo=0x30, scale_hi=0x48, p7f=0)
    gs_gu, gs_dn = 2.0e-3, 3.0e-3
    s_gu, s_dn = load_expert_slabs(gu, E, 2 * I, H, gs_gu), load_expert_slabs(dn, E, H, I, gs_dn)
    table = expert_table(s_gu, s_dn)
    t = 2
    picks = np.array([[3, 200, 17, 255, 0, 96, 41, 128], [200, 5, 6, 7, 250, 3, 64, 1]], np.int64)
    x = (normal_f32(5, 900, t * H) * np.float32(0.1)).reshape(t, H)
    hin = (normal_f32(5, 901, t * K * I) * np.float32(0.3)).reshape(t * K, I)
    p = eng.p
    gup = table[torch.from_numpy(picks.reshape(-1)).cuda(), 0].contiguous()
    dnp = table[torch.from_numpy(picks.reshape(-1)).cuda(), 1].contiguous()
    xd, hd = _dev(x), _dev(hin)
    h1 = torch.empty((t * K, 2 * I), dtype=torch.float32, device="cuda")
    launch_v(eng.k.f("gemv_fp4_ptrb"), *launch_dims("gemv_fp4_ptrb", 2 * I, H, t * K),
             [gup.data_ptr(), xd.data_ptr(), s_gu.gs.data_ptr(), h1.data_ptr(), p.i32(H), p.i32(K), p.i32(H), p.i32(2 * I)])
    h2 = torch.empty((t * K, I), dtype=torch.float32, device="cuda")
    launch_v(eng.k.f("moe_gate_up_silu"), *launch_dims("moe_gate_up_silu", I, H, t * K),
             [gup.data_ptr(), xd.data_ptr(), s_gu.gs.data_ptr(), h2.data_ptr(), p.i32(H), p.i32(K), p.i32(H), p.i32(I)])
    eo = torch.empty((t * K, H), dtype=torch.float32, device="cuda")
    launch_v(eng.k.f("gemv_fp4_ptrb"), *launch_dims("gemv_fp4_ptrb", H, I, t * K),
             [dnp.data_ptr(), hd.data_ptr(), s_dn.gs.data_ptr(), eo.data_ptr(), p.i32(I), p.i32(1), p.i32(I), p.i32(H)])
    eng.check()
    h1n, h2n, eon = h1.cpu().numpy(), h2.cpu().numpy(), eo.cpu().numpy()
    per_gu, per_dn = 2 * I * H // 64 * 36, H * I // 64 * 36
    for c in range(t * K):
        e = int(picks.reshape(-1)[c])
        wgu, wdn = gu[e * per_gu:(e + 1) * per_gu], dn[e * per_dn:(e + 1) * per_dn]
        r1 = orc.gemv(wgu, 2 * I, H, gs_gu, x[c // K])[0]
        assert rel_err(h1n[c], r1) <= TOL and gamma_ratio(h1n[c], wgu, 2 * I, H, gs_gu, x[c // K]) <= 1.0, c
        assert rel_err(h2n[c], orc.silu_mul(r1[None, :I], r1[None, I:])[0]) <= TOL, c
        assert rel_err(eon[c], orc.gemv(wdn, H, I, gs_dn, hin[c])[0]) <= TOL and gamma_ratio(eon[c], wdn, H, I, gs_dn, hin[c]) <= 1.0, c


def test_moe_layer_other_geometries_drawn_at_random(eng):
    """Eight routed layers with other expert counts, pick counts, widths and batch sizes (fixed seed), every launch
    sequence - five launches, three, two (router inside gate|up), grouped by expert - against the CPU path."""
    from crow_nest_amd.engine import MoeW, expert_table
    from crow_nest_amd.kernels import KernelGeo
    from crow_nest_amd.weights import load_expert_slabs
    g = np.random.default_rng(77)
    keep = eng.geo
    try:
        for case in range(8):
            E = int(g.choice([64, 128]))
            K = int(g.choice([1, 2, 3, 6, 8, 10]))
            H = 64 * int(g.integers(2, 13))
            I = 64 * int(g.integers(1, 7))
            t = int(g.integers(1, 8))
            print(f"case {case}: E={E} K={K} H={H} I={I} t={t}", flush=True)
            eng.set_geo(KernelGeo(experts=E, topk=K, hidden=H, inter=I))
            gu = random_nvfp4(300 + case, E * 2 * I, H, scale_lo=0x30, scale_hi=0x48, p7f=0)
            dn = random_nvfp4(400 + case, E * H, I, scale_lo=0x30, scale_hi=0x48, p7f=0)
            gs_gu, gs_dn = 2.0e-3, 3.0e-3
            s_gu, s_dn = load_expert_slabs(gu, E, 2 * I, H, gs_gu), load_expert_slabs(dn, E, H, I, gs_dn)
            moe = MoeW(s_gu, s_dn, expert_table(s_gu, s_dn))
            x = (normal_f32(15, case, t * H) * np.float32(0.1)).reshape(t, H)
            logits = normal_f32(16, case, t * E).reshape(t, E)
            ids_ref, w_ref, y_ref = orc.moe_layer(gu, gs_gu, dn, gs_dn, E, H, I, x, logits, K, threads=4)
            for fused in (False, True, "route", "grouped"):
                if fused == "grouped":
                    ids, wts, y, _ = eng.moe_run_grouped(moe, _dev(x), _dev(logits))
                else:
                    ids, wts, y = eng.moe_run(moe, _dev(x), _dev(logits), fused=fused)
                eng.check()
                assert np.array_equal(ids.cpu().numpy(), ids_ref), (case, fused)
                assert np.allclose(wts.cpu().numpy(), w_ref, rtol=2e-6, atol=0), (case, fused)
                assert rel_err(y.cpu().numpy(), y_ref, FLOOR_CHAINED) <= TOL, (case, fused)
    finally:
        eng.set_geo(keep)
    eng.check()


@pytest.mark.parametrize("t", [3, 24, 64])
def test_moe_layer_grouped_by_expert(eng, t):
    """Batches in which experts repeat: the plan is a stable sort of the combos by expert cut into tiles of at most four,
    and the layer's output matches the CPU path (which walks token by token)."""
    from crow_nest_amd.engine import MoeW, expert_table
    from crow_nest_amd.weights import load_expert_slabs
    E, H, I, K = 256, 2048, 512, 8
    print(f"case grouped moe t={t}", flush=True)
    gu = random_nvfp4(41, E * 2 * I, H, scale_lo=0x30, scale_hi=0x48, p7f=0)
    dn = random_nvfp4(42, E * H, I, scale_lo=0x30, scale_hi=0x48, p7f=0)
    gs_gu, gs_dn = 2.0e-3, 3.0e-3
    s_gu, s_dn = load_expert_slabs(gu, E, 2 * I, H, gs_gu), load_expert_slabs(dn, E, H, I, gs_dn)
    moe = MoeW(s_gu, s_dn, expert_table(s_gu, s_dn))
    x = (normal_f32(5, 100 + t, t * H) * np.float32(0.1)).reshape(t, H)
    logits = normal_f32(6, 100 + t, t * E).reshape(t, E)
    logits[:, :16] += np.float32(2.5)  # a few popular experts: long groups
    ids_ref, w_ref, y_ref = orc.moe_layer(gu, gs_gu, dn, gs_dn, E, H, I, x, logits, K, threads=8)
    ids, wts, y, (perm, tiles, n_tiles) = eng.moe_run_grouped(moe, _dev(x), _dev(logits))
    eng.check()
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    # the plan: perm = stable argsort of the expert ids; tiles cover every group in runs of at most four
    flat = ids_ref.reshape(-1)
    assert np.array_equal(perm.cpu().numpy(), np.argsort(flat, kind="stable").astype(np.int32))
    nt = int(n_tiles.item())
    tl = tiles.cpu().numpy()[:nt]
    want = []
    start = 0
    for e in range(E):
        c = int((flat == e).sum())
        for q in range(0, c, 4):
            want.append((e, start + q, min(4, c - q), 0))
        start += c
    assert tl.tolist() == [list(w_) for w_ in want]
    assert rel_err(y.cpu().numpy(), y_ref, FLOOR_CHAINED) <= TOL
    # the ungrouped sequence gives the same layer
    _, _, y2 = eng.moe_run(moe, _dev(x), _dev(logits), fused=True)
    assert rel_err(y2.cpu().numpy(), y_ref, FLOOR_CHAINED) <= TOL
    eng.check()


@pytest.mark.parametrize("inter,hdim", [(512, 2048), (448, 200), (320, 1000)])
def test_grouped_down_on_strips_of_two_groups_gives_the_bits_of_one_row_launches(eng, inter, hdim):
    """K in 257 .. 512 (the down slabs of this model: K = 512): moe_down_grouped runs its twin that stages a tile's activation
    rows once per block and streams runs of strips.  Every output row must be, bit for bit, what a one-row launch (gemv_nvfp4_w)
    gives on that combo's slab and activation row - the contract of every kernel for several rows - also with a partial last
    group (K = 448, 320), a row count that is no multiple of 16 or of a block's strips, and tiles of 1 .. 4 rows."""
    from crow_nest_amd.kernels import launch_dims, launch_v
    from crow_nest_amd.weights import load_expert_slabs
    E = 8
    print(f"case grouped down inter={inter} hdim={hdim}", flush=True)
    dn = random_nvfp4(910 + inter, E * hdim, inter, scale_lo=0x30, scale_hi=0x48, p7f=0)
    slabs = load_expert_slabs(dn, E, hdim, inter, 3.0e-3)
    ids = np.array([3, 1, 3, 0, 3, 7, 3, 1, 7, 3, 7, 5, 5, 5], dtype=np.int32)  # expert 3: five combos -> tiles of 4 + 1
    combos = ids.size
    perm = np.argsort(ids, kind="stable").astype(np.int32)
    tiles, start = [], 0
    for e in range(E):
        c = int((ids == e).sum())
        for q in range(0, c, 4):
            tiles.append((e, start + q, min(4, c - q), 0))
        start += c
    max_tiles = len(tiles) + 3  # blocks of tiles beyond the count leave at once
    tl = np.zeros((max_tiles, 4), dtype=np.int32)
    tl[:len(tiles)] = np.array(tiles, dtype=np.int32)
    table = torch.tensor([[0, slabs.ptr(e)] for e in range(E)], dtype=torch.int64, device=eng.dev)
    h = normal_f32(12, inter + hdim, combos * inter).reshape(combos, inter)
    hd = _dev(h)
    eo = torch.full((combos, hdim), float("nan"), dtype=torch.float32, device=eng.dev)
    p = eng.p
    dims = launch_dims("moe_down_grouped", hdim, inter, max_tiles)
    assert dims[3] == 256 and dims[0] == (hdim + 16 * 32 - 1) // (16 * 32) and dims[1] >> 24 == 8  # the twin's grid: 4 waves x 8 strips per block
    tl_d, nt_d, perm_d = _dev(tl), _dev(np.array([len(tiles)], dtype=np.int32)), _dev(perm)
    launch_v(eng.k.f("moe_down_grouped"), *dims,
             [tl_d.data_ptr(), nt_d.data_ptr(), perm_d.data_ptr(), table.data_ptr(), hd.data_ptr(), slabs.gs.data_ptr(), eo.data_ptr(), p.i32(inter),
              p.i32(hdim)])
    eng.check()
    got = eo.cpu().numpy()
    one = torch.empty((hdim,), dtype=torch.float32, device=eng.dev)
    d1 = launch_dims("gemv_nvfp4_w", hdim, inter, 1)
    rb = inter // 64 * 36
    for c in range(combos):
        e = int(ids[c])
        launch_v(eng.k.f("gemv_nvfp4_w"), *d1, [slabs.ptr(e), hd[c].data_ptr(), slabs.gs.data_ptr(), one.data_ptr(), p.i32(inter), p.i32(hdim)])
        eng.check()
        assert np.array_equal(one.cpu().numpy().view(np.uint32), got[c].view(np.uint32)), c
    ref = orc.gemv(dn[3 * hdim * rb:4 * hdim * rb], hdim, inter, 3.0e-3, h[2])[0]  # combo 2 picked expert 3
    assert rel_err(got[2], ref) <= TOL


@pytest.mark.parametrize("inter,hdim", [(512, 2048), (96, 1600), (48, 320)])
def test_grouped_gate_up_on_short_strips_gives_the_bits_of_per_combo_launches(eng, inter, hdim):
    """K up to 2048 (this model's gate|up slabs: K = 2048, eight groups per strip): moe_gate_up_silu_grouped runs its twin that
    stages a tile's activation rows once per block and streams gate strip, up strip, gate strip ... per wave.  Every row of h
    must be, bit for bit, what the per-combo kernel (moe_gate_up_silu) gives for that combo - also with a partial last group
    (K = 1600, 320), few rows, and tiles of 1 .. 4 rows."""
    from crow_nest_amd.kernels import launch_dims, launch_v
    from crow_nest_amd.weights import load_expert_slabs
    E, topk = 8, 2
    print(f"case grouped gate|up inter={inter} hdim={hdim}", flush=True)
    gu = random_nvfp4(930 + inter, E * 2 * inter, hdim, scale_lo=0x30, scale_hi=0x48, p7f=0)
    slabs = load_expert_slabs(gu, E, 2 * inter, hdim, 2.0e-3)
    ids = np.array([3, 1, 3, 0, 3, 7, 3, 1, 7, 3, 7, 5, 5, 5], dtype=np.int32)  # combo c belongs to token c // topk
    combos, t = ids.size, ids.size // topk
    perm = np.argsort(ids, kind="stable").astype(np.int32)
    tiles, start = [], 0
    for e in range(E):
        c = int((ids == e).sum())
        for q in range(0, c, 4):
            tiles.append((e, start + q, min(4, c - q), 0))
        start += c
    max_tiles = len(tiles) + 2
    tl = np.zeros((max_tiles, 4), dtype=np.int32)
    tl[:len(tiles)] = np.array(tiles, dtype=np.int32)
    table = torch.tensor([[slabs.ptr(e), 0] for e in range(E)], dtype=torch.int64, device=eng.dev)
    x = _dev((normal_f32(13, inter + hdim, t * hdim) * np.float32(0.3)).reshape(t, hdim))
    p = eng.p
    tl_d, nt_d, perm_d = _dev(tl), _dev(np.array([len(tiles)], dtype=np.int32)), _dev(perm)
    h = torch.full((combos, inter), float("nan"), dtype=torch.float32, device=eng.dev)
    dims = launch_dims("moe_gate_up_silu_grouped", inter, hdim, max_tiles)
    assert dims[1] >> 24 >= 1 and dims[3] in (256, 512)  # the twin's launch shape: strips per wave in the top byte
    launch_v(eng.k.f("moe_gate_up_silu_grouped"), *dims,
             [tl_d.data_ptr(), nt_d.data_ptr(), perm_d.data_ptr(), table.data_ptr(), x.data_ptr(), slabs.gs.data_ptr(), h.data_ptr(), p.i32(hdim),
              p.i32(topk), p.i32(hdim), p.i32(inter)])
    eng.check()
    ptrs = torch.tensor([slabs.ptr(int(e)) for e in ids], dtype=torch.int64, device=eng.dev)
    h1 = torch.full((combos, inter), float("nan"), dtype=torch.float32, device=eng.dev)
    launch_v(eng.k.f("moe_gate_up_silu"), *launch_dims("moe_gate_up_silu", inter, hdim, combos),
             [ptrs.data_ptr(), x.data_ptr(), slabs.gs.data_ptr(), h1.data_ptr(), p.i32(hdim), p.i32(topk), p.i32(hdim), p.i32(inter)])
    eng.check()
    assert np.array_equal(h.cpu().numpy().view(np.uint32), h1.cpu().numpy().view(np.uint32))
    assert np.isfinite(h.cpu().numpy()).all()


# ---------------------------------------------------------------- benchmark config 0 (dense GEMV [17408, 5120], f32 x) at full size

def test_config0_full_size(eng):
    rows, cols = 17408, 5120
    w, gs = quantized_normal(0, 0, rows, cols)
    x = normal_f32(0, 1, cols)
    f = _load(w, rows, cols, gs)
    y = eng.dense_proj(f, 1, _dev(x)).cpu().numpy()[0]
    eng.check()
    ref = orc.gemv(w, rows, cols, gs, x, threads=8)[0]
    assert rel_err(y, ref) <= TOL and rel_l2(y, ref) <= 1e-4
    for r0 in (0, 8704 - 256, rows - 512):
        assert gamma_rows(y[r0:r0 + 512], w, r0, 512, cols, gs, x) <= 1.0, r0
    # dequantised weights bit-exact on a slab of the full tensor
    from crow_nest_amd.weights import dequant
    d = dequant(f)[:256].cpu().numpy().reshape(-1)
    assert np.array_equal(d.view(np.uint32), orc.dequant(w[:256 * cols // 64 * 36], gs).view(np.uint32))


# ---------------------------------------------------------------- benchmark config 1 (gate | up + SiLU and down, M <= 4) at full size

def test_config1_full_size_properties(eng):
    """[17408, 5120] gate / up and [5120, 17408] down, the benchmark's weights and bf16 X, four token rows: sampled row slabs
    against the CPU path, every row of the four-row launch bit-identical to its own one-row launch, and the down
    projection exactly linear under power-of-two scaling."""
    from crow_nest_amd.engine import MlpW
    H, I, T = 5120, 17408, 4
    (wg, gg), (wu, gu), (wd, gd) = quantized_normal(0, 0, I, H), quantized_normal(0, 1, I, H), quantized_normal(0, 2, H, I)
    mlp = MlpW(_load(wg, I, H, gg), _load(wu, I, H, gu), _load(wd, H, I, gd))
    xb, xw = _bf16_dev(normal_f32(0, 3, T * H))
    xb, xw = xb.reshape(T, H).contiguous(), xw.reshape(T, H)
    h4 = eng.gate_up(mlp, T, xb)
    eng.check()
    h = h4.cpu().numpy()
    rb = H // 64 * 36
    for r0 in (0, 8704 - 64, I - 128):
        g_ref = orc.gemv(wg[r0 * rb:(r0 + 128) * rb], 128, H, gg, xw, threads=8)
        u_ref = orc.gemv(wu[r0 * rb:(r0 + 128) * rb], 128, H, gu, xw, threads=8)
        assert rel_err(h[:, r0:r0 + 128], orc.silu_mul(g_ref, u_ref)) <= TOL, r0
    for t in range(T):
        h1 = eng.gate_up(mlp, 1, xb[t:t + 1].contiguous()).cpu().numpy()
        assert np.array_equal(h1.view(np.uint32)[0], h.view(np.uint32)[t]), t
    # the two-row launch (its own bodies of the gate / up and down kernels): rows 1..2 of the four, bit for bit and against the CPU path
    h2 = eng.gate_up(mlp, 2, xb[1:3].contiguous())
    eng.check()
    assert np.array_equal(h2.cpu().numpy().view(np.uint32), h.view(np.uint32)[1:3])
    r0 = 8704 - 64
    assert rel_err(h2.cpu().numpy()[:, r0:r0 + 128], orc.silu_mul(orc.gemv(wg[r0 * rb:(r0 + 128) * rb], 128, H, gg, xw[1:3], threads=8),
                                                                   orc.gemv(wu[r0 * rb:(r0 + 128) * rb], 128, H, gu, xw[1:3], threads=8))) <= TOL
    # the gate product alone (bf16 X, four rows) inside the reference's own bound on sampled rows
    g4 = eng.proj_m(mlp.gate, T, xb).cpu().numpy()
    for r0 in (0, I - 256):
        assert gamma_rows(g4[:, r0:r0 + 256], wg, r0, 256, H, gg, xw) <= 1.0, r0
    y = eng.dense_proj(mlp.down, T, h4).cpu().numpy()
    eng.check()
    rbd = I // 64 * 36
    for r0 in (0, H - 256):
        assert rel_err(y[:, r0:r0 + 256], orc.gemv(wd[r0 * rbd:(r0 + 256) * rbd], 256, I, gd, h, threads=8)) <= TOL, r0
        assert gamma_rows(y[:, r0:r0 + 256], wd, r0, 256, I, gd, h) <= 1.0, r0
    y2 = eng.dense_proj(mlp.down, 2, h2).cpu().numpy()
    eng.check()
    assert np.array_equal(y2.view(np.uint32), y.view(np.uint32)[1:3])
    y8 = eng.dense_proj(mlp.down, T, (h4 * 8.0).contiguous()).cpu().numpy()
    assert np.array_equal(y8.view(np.uint32), (y * np.float32(8.0)).view(np.uint32))
    for t in (0, 3):
        y1 = eng.dense_proj(mlp.down, 1, h4[t:t + 1].contiguous()).cpu().numpy()
        assert np.array_equal(y1.view(np.uint32)[0], y.view(np.uint32)[t]), t


# ---------------------------------------------------------------- benchmark config 3 (lm_head [151936, 5120] + greedy argmax) at full size

def test_config3_full_size_head(eng):
    """[151936, 5120] head (random codes and scales: the encoder is not what is tested here): sampled row slabs against the
    CPU path, the fused argmax against the argmax of the logits the device wrote, fused and two-kernel forms equal."""
    rows, cols = 151936, 5120
    w = random_nvfp4(77, rows, cols, scale_lo=0x30, scale_hi=0x50, p7f=0)
    gs = 1.0e-3
    f = _load(w, rows, cols, gs)
    x = normal_f32(0, 5, cols)
    logits, idx = eng.lm_head_row(f, _dev(x), fused=True)
    eng.check()
    got = logits.cpu().numpy().reshape(-1)
    rb = cols // 64 * 36
    for r0 in (0, 75968 - 100, rows - 256):
        ref = orc.gemv(w[r0 * rb:(r0 + 256) * rb], 256, cols, gs, x, threads=8)[0]
        assert rel_err(got[r0:r0 + 256], ref) <= TOL, r0
        assert gamma_rows(got[r0:r0 + 256], w, r0, 256, cols, gs, x) <= 1.0, r0
    assert int(idx.item()) == orc.argmax_ref(got) == int(np.argmax(got))
    logits2, idx2 = eng.lm_head_row(f, _dev(x), fused=False)
    assert np.array_equal(logits2.cpu().numpy().reshape(-1).view(np.uint32), got.view(np.uint32))
    assert int(idx2.item()) == int(idx.item())
    eng.check()


# ---------------------------------------------------------------- batched GEMM on the matrix cores (config 4)

@pytest.mark.parametrize("kernel", ["gemm_nvfp4_bf16_m16", "gemm_nvfp4_bf16_m32", "gemm_nvfp4_bf16_m48", "gemm_nvfp4_bf16_m64", "gemm_nvfp4_bf16_m96",
                                    "gemm_nvfp4_bf16", "gemm_nvfp4_bf16_w48", "gemm_nvfp4_bf16_w64", "gemm_nvfp4_bf16_w80", "gemm_nvfp4_bf16_w96"])
@pytest.mark.parametrize("m,rows,cols", [(16, 320, 1024), (5, 100, 320), (17, 100, 320), (33, 256, 512), (128, 512, 2048), (200, 192, 5120)])
def test_gemm_bf16_against_the_cpu_path(eng, m, rows, cols, kernel):
    """Weights decode to exact bf16, X is bf16, products are exact in f32: only the summation order
    differs from the CPU path (which gets the exactly widened X)."""
    _gemm_case(eng, m, rows, cols, kernel)


def test_gemm_ragged_shapes_drawn_at_random(eng):
    """Sixteen (tokens, rows, columns) triples drawn with a fixed seed - partial row tiles, partial panels, partial token
    blocks - through the entry point the library picks and through one drawn at random."""
    g = np.random.default_rng(4242)
    names = ["gemm_nvfp4_bf16_m32", "gemm_nvfp4_bf16_m48", "gemm_nvfp4_bf16_m64", "gemm_nvfp4_bf16_m96", "gemm_nvfp4_bf16", "gemm_nvfp4_bf16_w48",
             "gemm_nvfp4_bf16_w64", "gemm_nvfp4_bf16_w80", "gemm_nvfp4_bf16_w96"]
    for case in range(16):
        m = int(g.integers(5, 300))
        rows = int(g.integers(1, 700))
        cols = 64 * int(g.integers(1, 50))
        forced = names[int(g.integers(0, len(names)))] if m > 16 else "gemm_nvfp4_bf16_m16"
        print(f"case {case}: m={m} rows={rows} cols={cols} forced={forced}", flush=True)
        w = random_nvfp4(500 + case, rows, cols)
        gs = 6.0e-4
        f = _load(w, rows, cols, gs)
        xb, xw = _bf16_dev(normal_f32(17, case, m * cols))
        ref = orc.gemv(w, rows, cols, gs, xw.reshape(m, cols), threads=8)
        for kernel in (None, forced):
            y = eng.gemm(f, m, xb.reshape(m, cols).contiguous(), kernel=kernel).cpu().numpy()
            eng.check()
            assert rel_err(y, ref, floor_of(y.size)) <= TOL, (case, kernel)
            assert gamma_ratio(y[:2], w, rows, cols, gs, xw.reshape(m, cols)[:2]) <= 1.0, (case, kernel)


def test_gemm_m16_full_size_cross_block_split(eng):
    """[17408, 5120] at 16 tokens: the K-split kernel's five column slices meet through the workspace."""
    _gemm_case(eng, 16, 17408, 5120, "gemm_nvfp4_bf16_m16")


def _gemm_case(eng, m, rows, cols, kernel):
    print(f"case m={m} rows={rows} cols={cols} {kernel}", flush=True)
    if kernel == "gemm_nvfp4_bf16_m16" and m > 16:
        from crow_nest_amd.kernels import launch_dims
        from crow_nest_amd.lib import CrowHipError
        with pytest.raises(CrowHipError):  # refused on the host, nothing launched
            launch_dims(kernel, rows, cols, m)
        return
    w = random_nvfp4(m * 7 + rows, rows, cols)
    gs = 6.0e-4
    f = _load(w, rows, cols, gs)
    xb, xw = _bf16_dev(normal_f32(7, m, m * cols))
    y = eng.gemm(f, m, xb.reshape(m, cols).contiguous(), kernel=kernel).cpu().numpy()
    eng.check()
    ref = orc.gemv(w, rows, cols, gs, xw.reshape(m, cols), threads=8)
    assert rel_err(y, ref, floor_of(y.size)) <= TOL
    assert gamma_ratio(y[:4], w, rows, cols, gs, xw.reshape(m, cols)[:4]) <= 1.0


@pytest.mark.parametrize("m", [512, 128, 384])
def test_gemm_full_size_sampled_rows(eng, m):
    """Benchmark config 4 (batched GEMM) at M = 512 and M = 128 on the full [17408, 5120] tensor; the CPU path checks 768 sampled rows."""
    rows, cols = 17408, 5120
    print(f"case m={m}", flush=True)
    w, gs = quantized_normal(0, 0, rows, cols)
    f = _load(w, rows, cols, gs)
    xb, xw = _bf16_dev(normal_f32(0, 40, m * cols))
    y = eng.gemm(f, m, xb.reshape(m, cols).contiguous()).cpu().numpy()
    eng.check()
    rb = cols // 64 * 36
    for r0 in (0, 8704 - 128, 17408 - 256):
        ref = orc.gemv(w[r0 * rb:(r0 + 256) * rb], 256, cols, gs, xw.reshape(m, cols), threads=8)
        assert rel_err(y[:, r0:r0 + 256], ref, floor_of(3 * ref.size)) <= TOL, r0
        assert gamma_rows(y[:8, r0:r0 + 256], w, r0, 256, cols, gs, xw.reshape(m, cols)[:8]) <= 1.0, r0
    # linearity, a size-independent property: rows of X scaled by powers of two scale Y exactly
    x2 = (xb.reshape(m, cols).float() * 4.0).to(torch.bfloat16).contiguous()
    y2 = eng.gemm(f, m, x2).cpu().numpy()
    assert np.array_equal(y2.view(np.uint32), (y * np.float32(4.0)).view(np.uint32))


# ---------------------------------------------------------------- a real container through the load path

def test_container_tensors_load_dequantise_and_multiply(eng):
    """Every NVFP4 tensor of the reference's container fixture: read from the file, repacked at load, dequantised
    bit-exactly, multiplied within tolerance; its gate / down pair run as one dense FFN."""
    import os

    from conftest import GOLDEN
    from crow_nest_amd.cnq import Cnq
    from crow_nest_amd.weights import dequant, load_fp4_cnq, unpack
    c = Cnq.open(os.path.join(GOLDEN, "synthetic-v2.cnq"))
    loaded = {}
    for t in c.tensors:
        if t.dtype != "nvfp4":
            continue
        print(f"case {t.name} {t.shape}", flush=True)
        raw = c.read_bytes(t)
        rows, cols = t.shape
        f = load_fp4_cnq(c, t.name, t.section)
        assert np.array_equal(unpack(f), raw)  # no 0x7F scale byte in this container: the round trip is the identity
        want = orc.dequant(raw, t.global_scale)
        assert np.array_equal(dequant(f).cpu().numpy().reshape(-1).view(np.uint32), want.view(np.uint32))
        x = normal_f32(11, len(loaded), 3 * cols).reshape(3, cols)
        y = eng.proj_m(f, 3, _dev(x)).cpu().numpy()
        assert rel_err(y, orc.gemv(raw, rows, cols, t.global_scale, x)) <= TOL
        loaded[t.name] = (f, raw, t)
    assert len(loaded) == 6
    # layers.0 gate_proj [128, 64] as gate AND up, layers.1 down_proj [64, 128] as down: a small dense FFN from the file
    from crow_nest_amd.engine import MlpW
    g, graw, gt = loaded["model.language_model.layers.0.mlp.gate_proj.weight"]
    u, uraw, ut = loaded["model.language_model.layers.0.linear_attn.in_proj_qkv.weight"]
    d, draw, dt = loaded["model.language_model.layers.1.mlp.down_proj.weight"]
    x = normal_f32(12, 0, 2 * 64).reshape(2, 64) * np.float32(40.0)
    y = eng.dense_ffn_w(MlpW(g, u, d), _dev(x), 2).cpu().numpy()
    ref = orc.ffn(graw, gt.global_scale, uraw, ut.global_scale, draw, dt.global_scale, 64, 128, x)
    assert rel_err(y, ref, FLOOR_CHAINED) <= TOL
    eng.check()
    c.close()


# ---------------------------------------------------------------- captured launch sequences

def test_captured_sequence_replays_match_eager_launches(eng):
    """The decode sequence gate/up+SiLU -> down -> lm_head with its argmax, captured once and replayed
    with new inputs, eager work and synchronisations in between: every replay equals the eager result bit for bit."""
    from crow_nest_amd.kernels import Graph, launch_dims, launch_v, sync
    H, I, V = 1024, 2816, 4000
    wg, wu, wd, wh = random_nvfp4(31, I, H), random_nvfp4(32, I, H), random_nvfp4(33, H, I), random_nvfp4(34, V, H)
    g_, u_, d_, h_ = _load(wg, I, H, 2e-3), _load(wu, I, H, 1.5e-3), _load(wd, H, I, 1.1e-3), _load(wh, V, H, 9e-4)
    p = eng.p
    x = torch.zeros(H, dtype=torch.float32, device="cuda")
    hbuf = torch.empty(I, dtype=torch.float32, device="cuda")
    y = torch.empty(H, dtype=torch.float32, device="cuda")
    logits = torch.empty(V, dtype=torch.float32, device="cuda")
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    seq = [("gemv_nvfp4_gu", launch_dims("gemv_nvfp4_gu", I, H), [g_.w_ptr, u_.w_ptr, x.data_ptr(), g_.gs_ptr, u_.gs_ptr, hbuf.data_ptr(), p.i32(H), p.i32(I)]),
           ("gemv_nvfp4_w", launch_dims("gemv_nvfp4_w", H, I), [d_.w_ptr, hbuf.data_ptr(), d_.gs_ptr, y.data_ptr(), p.i32(I), p.i32(H)]),
           ("gemv_nvfp4_w_argmax", launch_dims("gemv_nvfp4_w_argmax", V, H), [h_.w_ptr, y.data_ptr(), h_.gs_ptr, logits.data_ptr(), p.i32(H), p.i32(V), tok.data_ptr()])]

    def eager():
        for name, dims, vals in seq:
            launch_v(eng.k.f(name), *dims, vals)
        sync()
        torch.cuda.synchronize()
        return y.cpu().numpy().copy(), logits.cpu().numpy().copy(), int(tok.item())

    torch.cuda.synchronize()
    gr = Graph()
    with gr.capture():
        for name, dims, vals in seq:
            launch_v(eng.k.f(name), *dims, vals)
    for r in range(4):
        x.copy_(_dev(normal_f32(50, r, H) * np.float32(0.05)))
        ye, le, te = eager()
        y.zero_(); logits.zero_(); tok.zero_()  # eager work of the program's own between the replays
        torch.cuda.synchronize()
        gr.launch()
        gr.sync()
        assert np.array_equal(y.cpu().numpy().view(np.uint32), ye.view(np.uint32)), r
        assert np.array_equal(logits.cpu().numpy().view(np.uint32), le.view(np.uint32)), r
        assert int(tok.item()) == te == int(orc.argmax_ref(le)), r
    # and the replayed result is the CPU path's
    xr = normal_f32(50, 3, H) * np.float32(0.05)
    ref = orc.ffn(wg, 2e-3, wu, 1.5e-3, wd, 1.1e-3, H, I, xr.reshape(1, H))[0]
    assert rel_err(y.cpu().numpy(), ref, FLOOR_CHAINED) <= TOL
    gr.close()
    eng.check()


def test_launches_with_a_wrong_block_shape_are_refused(eng):
    """Blocks must be whole wavefronts (refused on the host); the one-row gate/up kernels need an even number of waves
    (refused by the kernel through the status word, nothing written)."""
    from crow_nest_amd.kernels import launch_dims, launch_v
    from crow_nest_amd.lib import CrowHipError
    rows, cols = 128, 512
    w = random_nvfp4(3, rows, cols)
    f = _load(w, rows, cols, 1.0e-3)
    x = _dev(normal_f32(1, 9, cols))
    y = torch.full((1, rows), 7.0, dtype=torch.float32, device="cuda")
    p = eng.p
    gx, gy, gz, bx = launch_dims("gemv_nvfp4_w", rows, cols)
    with pytest.raises(CrowHipError):
        launch_v(eng.k.f("gemv_nvfp4_w"), gx, gy, gz, 100, [f.w_ptr, x.data_ptr(), f.gs_ptr, y.data_ptr(), p.i32(cols), p.i32(rows)])
    gx, gy, gz, bx = launch_dims("gemv_nvfp4_gu", rows, cols)
    launch_v(eng.k.f("gemv_nvfp4_gu"), gx, gy, gz, 192, [f.w_ptr, f.w_ptr, x.data_ptr(), f.gs_ptr, f.gs_ptr, y.data_ptr(), p.i32(cols), p.i32(rows)])
    with pytest.raises(CrowHipError):
        eng.check()
    assert float(y.min()) == 7.0 == float(y.max())
    # the 32-token GEMM entry stages and reduces in LDS sized for four waves: a larger block is refused, nothing written
    xb = torch.zeros((20, cols), dtype=torch.bfloat16, device="cuda")
    yg = torch.full((20, rows), 7.0, dtype=torch.float32, device="cuda")
    gx, gy, gz, bx = launch_dims("gemm_nvfp4_bf16_m32", rows, cols, 20)
    for bad_bx in (512, 320):
        launch_v(eng.k.f("gemm_nvfp4_bf16_m32"), gx, gy, gz, bad_bx, [f.w_ptr, xb.data_ptr(), f.gs_ptr, yg.data_ptr(), p.i32(cols), p.i32(rows), p.i32(20)])
        with pytest.raises(CrowHipError) as ei:
            eng.check()
        assert ei.value.code == -7 and bool((yg == 7.0).all())
    eng.check()


def test_an_unsupported_geometry_is_refused_and_an_empty_pointer_table_is_not_followed(eng):
    """crow_hip_set_geo refuses an expert count the routing kernels do not take (on the host, nothing launched); and the
    routed kernels, handed a pointer table a refused routing launch would have left as zeros, report through the status
    word instead of reading weights at address zero."""
    from crow_nest_amd.kernels import KernelGeo, launch_dims, launch_v, set_geo
    from crow_nest_amd.lib import CrowHipError
    for bad in (KernelGeo(16, 4, 512, 256), KernelGeo(96, 4, 512, 256), KernelGeo(2048, 8, 512, 256), KernelGeo(256, 17, 512, 256), KernelGeo(64, 0, 512, 256)):
        with pytest.raises(CrowHipError) as ei:
            set_geo(bad)
        assert ei.value.code == -8  # CROW_ERR_GEO
    set_geo(eng.geo)
    H, I, K = eng.geo.hidden, eng.geo.inter, eng.geo.topk
    p = eng.p
    gs = torch.tensor([1e-3], dtype=torch.float32, device="cuda")
    zeros = torch.zeros(K, dtype=torch.int64, device="cuda")
    x = torch.zeros(H, dtype=torch.float32, device="cuda")
    h2 = torch.full((K, I), 7.0, dtype=torch.float32, device="cuda")
    y = torch.full((1, H), 7.0, dtype=torch.float32, device="cuda")
    wts = torch.ones(K, dtype=torch.float32, device="cuda")
    launch_v(eng.k.f("moe_gate_up_silu"), *launch_dims("moe_gate_up_silu", I, H, K),
             [zeros.data_ptr(), x.data_ptr(), gs.data_ptr(), h2.data_ptr(), p.i32(H), p.i32(K), p.i32(H), p.i32(I)])
    with pytest.raises(CrowHipError) as ei:
        eng.check()
    assert ei.value.code == -8 and float(h2.min()) == 7.0 == float(h2.max())
    launch_v(eng.k.f("gemv_fp4_ptrb"), *launch_dims("gemv_fp4_ptrb", 2 * I, H, K),
             [zeros.data_ptr(), x.data_ptr(), gs.data_ptr(), torch.empty((K, 2 * I), device="cuda").data_ptr(), p.i32(H), p.i32(K), p.i32(H), p.i32(2 * I)])
    with pytest.raises(CrowHipError) as ei:
        eng.check()
    assert ei.value.code == -8
    launch_v(eng.k.f("moe_down_combine"), *launch_dims("moe_down_combine", H, I, 1),
             [zeros.data_ptr(), h2.data_ptr(), gs.data_ptr(), wts.data_ptr(), y.data_ptr(), p.i32(I), p.i32(H)])
    with pytest.raises(CrowHipError) as ei:
        eng.check()
    assert ei.value.code == -8 and float(y.min()) == 7.0 == float(y.max())  # y += 0 from every combo
    # the kernels that take their slabs from the expert TABLE: a table whose entries are zeros is not followed either
    E = eng.geo.experts
    table0 = torch.zeros((E, 2), dtype=torch.int64, device="cuda")
    tiles = torch.tensor([[3, 0, 2, 0]], dtype=torch.int32, device="cuda")
    n_tiles = torch.ones(1, dtype=torch.int32, device="cuda")
    perm = torch.tensor([1, 0], dtype=torch.int32, device="cuda")
    xk = torch.zeros((1, H), dtype=torch.float32, device="cuda")
    eo = torch.full((K, H), 7.0, dtype=torch.float32, device="cuda")
    launch_v(eng.k.f("moe_gate_up_silu_grouped"), *launch_dims("moe_gate_up_silu_grouped", I, H, 1),
             [tiles.data_ptr(), n_tiles.data_ptr(), perm.data_ptr(), table0.data_ptr(), xk.data_ptr(), gs.data_ptr(), h2.data_ptr(),
              p.i32(H), p.i32(K), p.i32(H), p.i32(I)])
    with pytest.raises(CrowHipError) as ei:
        eng.check()
    assert ei.value.code == -8 and float(h2.min()) == 7.0 == float(h2.max())
    launch_v(eng.k.f("moe_down_grouped"), *launch_dims("moe_down_grouped", H, I, 1),
             [tiles.data_ptr(), n_tiles.data_ptr(), perm.data_ptr(), table0.data_ptr(), h2.data_ptr(), gs.data_ptr(), eo.data_ptr(), p.i32(I), p.i32(H)])
    with pytest.raises(CrowHipError) as ei:
        eng.check()
    assert ei.value.code == -8 and float(eo.min()) == 7.0 == float(eo.max())
    logits = _dev(normal_f32(6, 77, E).reshape(1, E))
    ids = torch.full((1, K), -1, dtype=torch.int32, device="cuda")
    wr = torch.zeros((1, K), dtype=torch.float32, device="cuda")
    dn = torch.zeros((1, K), dtype=torch.int64, device="cuda")
    launch_v(eng.k.f("moe_route_gate_up_silu"), *launch_dims("moe_route_gate_up_silu", I, H, K),
             [logits.data_ptr(), table0.data_ptr(), xk.data_ptr(), gs.data_ptr(), h2.data_ptr(), ids.data_ptr(), wr.data_ptr(), dn.data_ptr(),
              p.i32(H), p.i32(H), p.i32(I)])
    with pytest.raises(CrowHipError) as ei:
        eng.check()
    assert ei.value.code == -8 and float(h2.min()) == 7.0 == float(h2.max())
    # the host mirror refuses a table that does not cover the geometry's experts before anything is launched
    from crow_nest_amd.engine import MoeW
    from crow_nest_amd.weights import ExpertSlabs
    few = ExpertSlabs(torch.zeros(16, dtype=torch.uint8, device="cuda"), gs, E // 2, 2 * I, H, 8)
    few_dn = ExpertSlabs(torch.zeros(16, dtype=torch.uint8, device="cuda"), gs, E // 2, H, I, 8)
    bad = MoeW(few, few_dn, torch.zeros((E // 2, 2), dtype=torch.int64, device="cuda"))
    for run in (lambda: eng.moe_run(bad, xk, logits), lambda: eng.moe_run_grouped(bad, xk, logits), lambda: eng.router(logits, bad)):
        with pytest.raises(ValueError, match="experts"):
            run()
    eng.check()


def test_verify_kernels_refuse_more_than_four_rows(eng):
    """The reference's verify kernels take at most NVFP4_MMAX = 4 rows (kernels_p2.rs:397-400); a launch with m = 5 writes
    nothing and reports a shape error through the status word instead of computing four rows silently."""
    from crow_nest_amd.kernels import launch_dims, launch_v, status
    from crow_nest_amd.lib import CrowHipError
    rows, cols = 128, 512
    f = _load(random_nvfp4(61, rows, cols), rows, cols, 1e-3)
    x = torch.zeros(5 * cols, dtype=torch.float32, device="cuda")
    y = torch.full((5 * rows,), 7.0, dtype=torch.float32, device="cuda")
    p = eng.p
    with pytest.raises(CrowHipError) as ei:  # asked for by its own name, five rows are refused on the host
        launch_dims("gemv_nvfp4_wm", rows, cols, 5)
    assert ei.value.code == -7  # CROW_ERR_SHAPE
    # dims bound to four rows or to one row, and dims that leave the count to the device word (z = 0), the word behind m_p
    # saying five: a bound launch refuses because the word differs from its count, the unbound one because five is too many
    for z in (4, 1, 0):
        launch_v(eng.k.f("gemv_nvfp4_wm"), *launch_dims("gemv_nvfp4_wm", rows, cols, z), [f.w_ptr, x.data_ptr(), f.gs_ptr, y.data_ptr(), p.i32(cols), p.i32(rows), p.i32(5)])
        with pytest.raises(CrowHipError) as ei:
            status()
        assert ei.value.code == -7
        assert bool((y == 7.0).all())
    # and a launch whose dims were made for another K stores nothing either
    launch_v(eng.k.f("gemv_nvfp4_wm"), *launch_dims("gemv_nvfp4_wm", rows, cols // 2, 2), [f.w_ptr, x.data_ptr(), f.gs_ptr, y.data_ptr(), p.i32(cols), p.i32(rows), p.i32(2)])
    with pytest.raises(CrowHipError) as ei:
        status()
    assert ei.value.code == -7 and bool((y == 7.0).all())
    eng.check()


# ---------------------------------------------------------------- BF16 keeps

@pytest.mark.parametrize("rows,cols,t", [(256, 2048, 1), (256, 2048, 4), (37, 320, 3), (1000, 2560, 1), (64, 10240, 2), (5, 8, 1)])
def test_bf16_keep_gemv(eng, rows, cols, t):
    print(f"case rows={rows} cols={cols} t={t}", flush=True)
    w32 = normal_f32(70, rows, rows * cols) * np.float32(0.05)
    w_bits = orc.f32_to_bf16_bits(w32).reshape(rows, cols)
    x = normal_f32(71, t, t * cols).reshape(t, cols)
    wd = torch.from_numpy(w_bits.view(np.int16)).cuda().view(torch.bfloat16)
    ref = orc.gemv_bf16(w_bits, rows, cols, x)
    wf = orc.bf16_bits_to_f32(w_bits).astype(np.float64)
    bound = orc.gamma(16 * (cols + 6)) * (np.abs(x.astype(np.float64)) @ np.abs(wf).T)  # gamma(n) of the oracle counts n / 16 + 10 steps
    xd = _dev(x)
    for waves_per_row in (0, 1, 4):  # the library's choice, one wave per row, a block of four waves per row
        y = eng._keep_proj("gemv_bf16_w", wd, t, xd, None, waves_per_row).cpu().numpy()
        eng.check()
        assert rel_err(y, ref) <= TOL, waves_per_row
        assert np.all(np.abs(y.astype(np.float64) - ref.astype(np.float64)) <= bound + 1e-30), waves_per_row



def test_bf16_keep_gemv_under_the_block_per_row_names(eng):
    """gemv_bf16 (one token) and gemv_bf16_b are the same product under the reference's other two names: same bits."""
    rows, cols, t = 300, 2560, 3
    w_bits = orc.f32_to_bf16_bits(normal_f32(72, 1, rows * cols) * np.float32(0.05)).reshape(rows, cols)
    x = normal_f32(73, t, t * cols).reshape(t, cols)
    wd = torch.from_numpy(w_bits.view(np.int16)).cuda().view(torch.bfloat16)
    y = eng.bf16_proj(wd, t, _dev(x)).cpu().numpy()
    yb = eng.bf16_proj(wd, t, _dev(x), kernel="gemv_bf16_b").cpu().numpy()
    y1 = eng.bf16_proj(wd, 1, _dev(x[1]), kernel="gemv_bf16").cpu().numpy()
    assert np.array_equal(y.view(np.uint32), yb.view(np.uint32)) and np.array_equal(y1.view(np.uint32)[0], y.view(np.uint32)[1])
    assert rel_err(y, orc.gemv_bf16(w_bits, rows, cols, x)) <= TOL
    from crow_nest_amd.lib import CrowHipError
    with pytest.raises(CrowHipError):  # the one-token name takes one token
        eng.bf16_proj(wd, 2, _dev(x[:2]), kernel="gemv_bf16")
    # gemv_bf16_ws: the sigmoid at the store; gemv_bf16_bs: two tensors into one [t][2 rows] buffer
    ys = eng.bf16_proj(wd, t, _dev(x), kernel="gemv_bf16_ws").cpu().numpy()
    want = (np.float32(1.0) / (np.float32(1.0) + np.exp(-y, dtype=np.float32))).astype(np.float32)
    assert np.max(np.abs(ys - want)) <= 2e-7  # expf in the last place; the sums are the plain kernel's
    both = torch.full((t, 2 * rows + 8), 7.0, dtype=torch.float32, device="cuda")
    eng.bf16_proj_strided(wd, t, _dev(x), both, 2 * rows + 8)
    eng.bf16_proj_strided(wd, t, _dev(x), both.view(-1)[rows:], 2 * rows + 8)
    got = both.cpu().numpy()
    assert np.array_equal(got[:, :rows].view(np.uint32), y.view(np.uint32)) and np.array_equal(got[:, rows:2 * rows].view(np.uint32), y.view(np.uint32))
    assert bool((got[:, 2 * rows:] == 7.0).all())
    eng.check()


@pytest.mark.parametrize("rows,cols,t", [(256, 2560, 1), (256, 2560, 4), (37, 20, 3), (288, 4096, 2), (5, 4, 1), (1000, 1028, 1)])
def test_f32_keep_gemv_router_projection(eng, rows, cols, t):
    """gemv_b: f32 weights (the router), against the exact dot product within the f32 summation bound, and against the
    reference's own summation order within the tolerance; then the logits feed the router."""
    print(f"case rows={rows} cols={cols} t={t}", flush=True)
    w = normal_f32(74, rows, rows * cols).reshape(rows, cols) * np.float32(0.05)
    x = normal_f32(75, t, t * cols).reshape(t, cols)
    ref = orc.gemv_f32w(w, rows, cols, x)
    ref_order = orc.gemv_f32w_reference_order(w, rows, cols, x)
    bound = orc.gamma(16 * (cols + 6)) * (np.abs(x.astype(np.float64)) @ np.abs(w.astype(np.float64)).T)
    wd, xd = _dev(w), _dev(x)
    for waves_per_row in (0, 1, 4):  # the library's choice, one wave per row, a block of four waves per row
        y = eng._keep_proj("gemv_b", wd, t, xd, None, waves_per_row).cpu().numpy()
        eng.check()
        assert rel_err(y, ref) <= TOL, waves_per_row
        assert rel_err(y, ref_order) <= TOL, waves_per_row
        assert np.all(np.abs(y.astype(np.float64) - ref.astype(np.float64)) <= bound + 1e-30), waves_per_row
    assert np.array_equal(eng.f32_proj(wd, t, xd).cpu().numpy(), eng._keep_proj("gemv_b", wd, t, xd, None, 0).cpu().numpy())


# ---------------------------------------------------------------- the ABI from plain C

def test_c_abi_from_a_plain_c_program():
    """tests/c_abi/c_abi_gemv.c (gcc, no Python or torch in the process): init, lookup, alloc, upload, repack, launch with the
    library's dims, status, download - and the result within tolerance of the CPU oracle."""
    import os
    import subprocess

    from conftest import ROOT
    exe = os.path.join(ROOT, "tests", "c_abi", "c_abi_gemv")
    if not os.path.exists(exe):
        subprocess.run(["make", "-C", os.path.dirname(exe)], check=True, capture_output=True)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0 and "c_abi ok" in r.stdout

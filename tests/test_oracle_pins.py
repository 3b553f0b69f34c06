"""Pins the CPU oracle before anything is compared with it.

Every check here is independent of the oracle's own formulae: reference-held fixtures
(synthetic-v2.cnq, fp8-e4m3fn-lut.tsv, glm5 dense-y.f32 + manifest sha256s), closed forms written
a second way (numpy f64), invariants of the format, and brute force on tiny inputs.  The shapes
and seeds of the GEMV checks are the ones engine/src/cpu_nvfp4.rs:570-727 uses.
"""
import hashlib
import json
import os
import struct

import numpy as np
import pytest

from conftest import GOLDEN
from oracle import oracle as orc
from refgen import SplitMix64, lcg_bf16_tensors, scale_mix, synth_nvfp4

MAG = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


# ---------------------------------------------------------------- format

def test_e2m1_closed_form():
    for n in range(16):
        want = np.float32(-MAG[n & 7] if n & 8 else MAG[n & 7])
        got = np.float32(orc.e2m1(n))
        assert got.view(np.uint32) == want.view(np.uint32), n  # -0.0 for code 8


def test_ue4m3_matches_the_torch_e4m3fn_table_the_reference_holds():
    rows = [l.split("\t") for l in open(os.path.join(GOLDEN, "fp8-e4m3fn-lut.tsv")) if not l.startswith("#")]
    table = {int(c): b.strip() for c, b in rows}
    for code in range(127):  # 127 is NaN in e4m3fn; ue4m3 reads it as 480
        bits = np.float32(orc.ue4m3(code)).view(np.uint32)
        assert f"{int(bits):08x}" == table[code], code
    assert orc.ue4m3(0x7F) == 480.0 and orc.ue4m3(0x7E) == 448.0
    for b in range(128):  # bit 7 is ignored
        assert orc.ue4m3(b | 0x80) == orc.ue4m3(b)
    prev = 0.0
    for b in range(1, 0x80):  # strictly monotonic ladder (converter/src/main.rs:2455-2463)
        v = orc.ue4m3(b)
        assert v > prev and np.isfinite(v)
        prev = v


def test_scale_lut_applies_the_0x7f_rule_only_to_0x7f():
    gs = np.float32(3.0517578e-5)
    lut = orc.scale_lut(float(gs))
    for b in range(256):
        e, m = (b >> 3) & 15, b & 7
        u = m * 2.0 ** -9 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
        want = np.float32(448.0 if b == 0x7F else u) * gs
        assert lut[b].view(np.uint32) == np.float32(want).view(np.uint32), hex(b)
    assert lut[0xFF] == np.float32(480.0) * gs


# ---------------------------------------------------------------- encoder + dequant vs the reference's container fixture

def _cnq_index():
    raw = open(os.path.join(GOLDEN, "synthetic-v2.cnq"), "rb").read()
    assert raw[:4] == b"CNQ1"
    n = struct.unpack("<Q", raw[-8:])[0]
    idx = json.loads(raw[-8 - n:-8])
    return raw, idx


def test_ceil_encoder_reproduces_the_reference_container_byte_for_byte():
    raw, idx = _cnq_index()
    src = lcg_bf16_tensors()
    seen = 0
    for t in idx["tensors"]:
        if t["dtype"] != "nvfp4":
            continue
        seen += 1
        at = idx["blob_offset"] + t["offset"]
        want = np.frombuffer(raw[at:at + t["len"]], np.uint8)
        got, gs = orc.quantize_ceil(src[t["name"]])
        assert got.size == want.size == orc.byte_len(*t["shape"])
        assert np.array_equal(got, want), t["name"]
        assert np.float32(gs) == np.float32(t["global_scale"]), t["name"]
    assert seen == 6


def test_dequant_of_the_reference_container_is_within_one_step_of_its_source():
    raw, idx = _cnq_index()
    src = lcg_bf16_tensors()
    for t in idx["tensors"]:
        if t["dtype"] != "nvfp4":
            continue
        at = idx["blob_offset"] + t["offset"]
        blocks = np.frombuffer(raw[at:at + t["len"]], np.uint8)
        gs = float(np.float32(t["global_scale"]))
        w = orc.dequant(blocks, gs)
        v = src[t["name"]]
        scales = orc.scale_lut(gs)[blocks.reshape(-1, 36)[:, :4]].reshape(-1)
        step = np.repeat(scales, 16)
        assert np.all(np.abs(w - v) <= step * (1 + 1e-6))  # ceil mode: error <= one scale step
        nz = w != 0
        assert np.all(np.sign(w[nz]) == np.sign(v[nz]))
        assert np.all(np.abs(v) <= 6 * step * (1 + 1e-6))  # never clips
        # no 0x7F in this fixture: both decodes agree
        assert np.array_equal(w.view(np.uint32), orc.dequant(blocks, gs, rule=False).view(np.uint32))


def test_dequant_closed_form_every_byte():
    # all 256 scale bytes x all 256 code bytes, f64 closed form written independently
    blocks = np.zeros((256 * 2, 36), np.uint8)
    for s in range(256):
        blocks[2 * s, :4] = s
        blocks[2 * s + 1, :4] = s
        blocks[2 * s, 4:] = np.arange(0, 32)
        blocks[2 * s + 1, 4:] = np.arange(224, 256)
    blocks[:, 4:] = (blocks[:, 4:].astype(int) * 37 + np.arange(512)[:, None]) % 256
    gs = np.float32(1.7e-3)
    for rule in (True, False):
        w = orc.dequant(blocks.reshape(-1), float(gs), rule=rule).reshape(512, 64)
        for bi in range(0, 512, 7):
            blk = blocks[bi]
            for idx in range(64):
                sc = int(blk[idx // 16])
                if rule and sc == 0x7F:
                    sc = 0x7E
                e, m = (sc >> 3) & 15, sc & 7
                u = m * 2.0 ** -9 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
                s = np.float32(np.float32(u) * gs)
                nib = (int(blk[4 + idx // 2]) >> (4 * (idx % 2))) & 15
                want = np.float32(np.float32(-MAG[nib & 7] if nib & 8 else MAG[nib & 7]) * s)
                assert w[bi, idx].view(np.uint32) == want.view(np.uint32)


def test_encoder_invariants_on_random_blocks():
    g = np.random.default_rng(7)
    v = (g.standard_normal(64 * 512) * g.choice([1e-4, 0.02, 3.0], size=64 * 512)).astype(np.float32)
    v[:64] = 0.0  # an all-zero block: scale byte 0, codes 0
    blocks, gs = orc.quantize_ceil(v)
    assert np.all(blocks[:36] == 0)
    w = orc.dequant(blocks, gs, rule=False)
    sc = orc.ue4m3
    scales = np.array([sc(int(b)) for b in blocks.reshape(-1, 36)[:, :4].reshape(-1)], np.float32) * np.float32(gs)
    step = np.repeat(scales, 16)
    assert np.all(np.abs(v) <= 6 * step * (1 + 1e-6))
    assert np.all(np.abs(w - v) <= step * (1 + 1e-6))
    amax = np.abs(v).reshape(-1, 16).max(1)
    assert np.float32(gs) == np.float32(np.float32(amax.max() / np.float32(6.0)) / np.float32(448.0))


# ---------------------------------------------------------------- GEMV arithmetic

def _xs(rng, n, a=2.0):
    return rng.f(n, a)


def _worst_ratio(y, yr, ab, cols):
    g = orc.gamma(cols)
    return float(np.max(np.abs(y.astype(np.float64) - yr) / np.maximum(g * ab, np.finfo(np.float64).tiny)))


def _f64_reference(w, rows, cols, gs, x, rule=True):
    """Independent numpy f64 dequantise-then-dot (not the oracle's own f64 routine)."""
    blk = np.asarray(w, np.uint8).reshape(rows, cols // 64, 36)
    sc = blk[:, :, :4].astype(np.int64)
    if rule:
        sc = np.where(sc == 0x7F, 0x7E, sc)
    e, m = (sc >> 3) & 15, sc & 7
    u = np.where(e == 0, m * 2.0 ** -9, (1 + m / 8.0) * 2.0 ** (e.astype(np.float64) - 7))
    s = (u.astype(np.float32) * np.float32(gs)).astype(np.float64)  # the engine's f32 scale
    codes = blk[:, :, 4:]
    nib = np.stack([codes & 15, codes >> 4], -1).reshape(rows, cols // 64, 64)
    mag = np.array(MAG)[nib & 7] * np.where(nib & 8, -1.0, 1.0)
    wd = (mag.reshape(rows, cols // 64, 4, 16) * s[..., None]).reshape(rows, cols)
    xv = np.asarray(x, np.float32).reshape(-1, cols).astype(np.float64)
    return xv @ wd.T, np.abs(xv) @ np.abs(wd).T


def test_gemv_holds_the_fp32_bound_on_the_reference_test_shapes():
    rng = SplitMix64(173)
    for rows, cols in [(37, 256), (16, 2048), (9, 4096)]:
        w = synth_nvfp4(rng, rows, cols, scale_mix)
        gs = 1.7e-3
        for t in [1, 2, 3, 5, 8]:
            x = _xs(rng, t * cols)
            yr, ab = _f64_reference(w, rows, cols, gs, x)
            yo, ao = orc.gemv_f64(w, rows, cols, gs, x)
            assert np.allclose(yo, yr, rtol=1e-12, atol=0) or np.max(np.abs(yo - yr)) <= 1e-12 * np.max(ab)
            for path in (0, 1):
                y = orc.gemv(w, rows, cols, gs, x, threads=3, path=path)
                assert _worst_ratio(y, yr, ab, cols) <= 1.0, (rows, cols, t, path)


def test_gemv_avx2_equals_scalar_bits_for_every_scale_byte_and_thread_count():
    rng = SplitMix64(0xC0FFEE)
    rows, cols = 41, 1024
    w = synth_nvfp4(rng, rows, cols, lambda r: int(r.bytes(1)[0]))
    gs = 2.3e-4
    for t in [1, 2, 3, 5, 8]:
        x = _xs(rng, t * cols)
        s1 = orc.gemv(w, rows, cols, gs, x, threads=1, path=0).view(np.uint32)
        for th in (1, 3, 8):
            assert np.array_equal(orc.gemv(w, rows, cols, gs, x, threads=th, path=0).view(np.uint32), s1)
            assert np.array_equal(orc.gemv(w, rows, cols, gs, x, threads=th, path=1).view(np.uint32), s1)
        yr, ab = _f64_reference(w, rows, cols, gs, x)
        assert _worst_ratio(s1.view(np.float32), yr, ab, cols) <= 1.0


def test_gemv_brute_force_in_the_documented_order():
    """A pure-python restatement of the 8-lane order on a tiny case, each op rounded to f32."""
    rng = SplitMix64(5)
    rows, cols = 3, 128
    w = synth_nvfp4(rng, rows, cols, scale_mix)
    gs = np.float32(9.5e-4)
    x = _xs(rng, 2 * cols).reshape(2, cols)
    lut = orc.scale_lut(float(gs))
    f = np.float32
    for r in range(rows):
        row = w[r * 72:(r + 1) * 72]
        for t in range(2):
            acc = [f(0)] * 8
            for b in range(2):
                blk = row[b * 36:(b + 1) * 36]
                for sb in range(4):
                    s = lut[blk[sb]]
                    for l in range(8):
                        c = int(blk[4 + sb * 8 + l])
                        lo = f(-MAG[c & 7] if c & 8 else MAG[c & 7])
                        hi = f(-MAG[(c >> 4) & 7] if c & 0x80 else MAG[(c >> 4) & 7])
                        p = f(f(lo * x[t, b * 64 + sb * 16 + 2 * l]) + f(hi * x[t, b * 64 + sb * 16 + 2 * l + 1]))
                        acc[l] = f(acc[l] + f(p * s))
            want = f(0)
            for l in range(8):
                want = f(want + acc[l])
            for path in (0, 1):
                got = orc.gemv(w, rows, cols, float(gs), x, path=path)[t, r]
                assert got.view(np.uint32) == want.view(np.uint32)


def test_scale_rule_is_the_slab_rule():
    rng = SplitMix64(0x7F)
    rows, cols = 12, 512

    def sc(r):
        return 0x7F if (int(r.bytes(1)[0]) & 1) == 0 else 0x70 + (int(r.bytes(1)[0]) & 7)

    w = synth_nvfp4(rng, rows, cols, sc, code_mask=0x77)
    gs = 9.5e-4
    x = np.abs(rng.f(2 * cols, 1.0)) + np.float32(0.01)
    y448, ab448 = _f64_reference(w, rows, cols, gs, x, rule=True)
    y480, ab480 = _f64_reference(w, rows, cols, gs, x, rule=False)
    g = orc.gamma(cols)
    for path in (0, 1):
        y = orc.gemv(w, rows, cols, gs, x, threads=2, path=path)
        assert _worst_ratio(y, y448, ab448, cols) <= 1.0
        assert np.all(np.abs(y.astype(np.float64) - y480) > g * ab480)
    clean = w.copy().reshape(-1, 36)
    clean[:, :4][clean[:, :4] == 0x7F] = 0x7E
    assert np.array_equal(orc.gemv(clean.reshape(-1), rows, cols, gs, x).view(np.uint32),
                          orc.gemv(w, rows, cols, gs, x).view(np.uint32))


def test_shapes_are_checked():
    b = np.zeros(orc.byte_len(3, 128), np.uint8)
    orc.gemv(b, 3, 128, 1.0, np.zeros(128, np.float32))
    with pytest.raises(ValueError):
        orc.gemv(b, 3, 96, 1.0, np.zeros(96, np.float32))
    with pytest.raises(ValueError):
        orc.gemv(b[1:], 3, 128, 1.0, np.zeros(128, np.float32))


def test_expert_ffn_against_f64_end_to_end():
    rng = SplitMix64(0xF00D)
    h, i = 192, 128
    gb, ub, db = (synth_nvfp4(rng, i, h, scale_mix), synth_nvfp4(rng, i, h, scale_mix), synth_nvfp4(rng, h, i, scale_mix))
    gs = [2.1e-3, 1.9e-3, 2.6e-3]
    for t in (1, 2, 5):
        x = _xs(rng, t * h)
        y = orc.ffn(gb, gs[0], ub, gs[1], db, gs[2], h, i, x, path=0)
        g = orc.gemv(gb, i, h, gs[0], x, path=0)
        u = orc.gemv(ub, i, h, gs[1], x, path=0)
        hk = orc.silu_mul(g, u)
        # the activation in f32: g / (1 + exp(-g)) * u, checked against f64 to a few ulp
        h64 = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u.astype(np.float64)
        assert np.all(np.abs(hk - h64) <= 4e-7 * np.abs(h64) + 1e-30)
        assert np.array_equal(orc.gemv(db, h, i, gs[2], hk, path=0).view(np.uint32), y.view(np.uint32))
        yr, ab = _f64_reference(db, h, i, gs[2], hk)
        assert _worst_ratio(y, yr, ab, i) <= 1.0
        g64, _ = _f64_reference(gb, i, h, gs[0], x)
        u64, _ = _f64_reference(ub, i, h, gs[1], x)
        hh = g64 / (1 + np.exp(-g64)) * u64
        want, mag = _f64_reference(db, h, i, gs[2], hh.astype(np.float32))  # f32 cast error << 1e-4
        assert np.all(np.abs(y - want) <= 1e-4 * mag)
        for th in (1, 3, 8):
            for path in (0, 1):
                y2 = orc.ffn(gb, gs[0], ub, gs[1], db, gs[2], h, i, x, threads=th, path=path)
                assert np.array_equal(y2.view(np.uint32), y.view(np.uint32))


# ---------------------------------------------------------------- the torch golden the reference holds

def _sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def glm5_dense_inputs():
    """The dense FFN inputs of engine/src/glm5_moe.rs:2385-2410 (`synth`), by stream position."""
    H, E, SH, DI = 4096, 288, 2048, 12288
    rng = SplitMix64(0x01646105)
    rng.skip(E * H)  # router weights (bf16)
    bias = rng.f(E, 0.09)

    def nvfp4(rows, cols):
        n = rows * cols // 64 * 36
        d = rng.next(n)
        out = (d & np.uint64(0xFF)).astype(np.uint8).reshape(-1, 36)
        out[:, :4] = (0x30 + (d.reshape(-1, 36)[:, :4] % np.uint64(16))).astype(np.uint8)
        return out.reshape(-1)

    shared = [nvfp4(SH, H), nvfp4(SH, H), nvfp4(H, SH)]
    dense = [nvfp4(DI, H), nvfp4(DI, H), nvfp4(H, DI)]
    x_route = rng.f(64 * H, 0.17)
    x_moe = rng.f(4 * H, 0.17)
    x_dense = rng.f(2 * H, 0.17)
    return dict(bias=bias, shared=shared, dense=dense, x_route=x_route, x_moe=x_moe, x_dense=x_dense)


def test_dense_ffn_matches_the_torch_golden_the_reference_holds():
    man = json.load(open(os.path.join(GOLDEN, "glm5-moe-manifest.json")))
    s = glm5_dense_inputs()
    sha = man["inputs_sha256"]
    assert _sha(s["bias"]) == sha["bias.f32"]
    for nm, a in zip(("gate", "up", "down"), s["shared"]):
        assert _sha(a) == sha[f"shared_{nm}.nvfp4"]
    for nm, a in zip(("gate", "up", "down"), s["dense"]):
        assert _sha(a) == sha[f"dense_{nm}.nvfp4"]
    assert _sha(s["x_route"]) == sha["x_route.f32"]
    assert _sha(s["x_moe"]) == sha["x_moe.f32"]
    assert _sha(s["x_dense"]) == sha["x_dense.f32"]
    golden = np.fromfile(os.path.join(GOLDEN, "glm5-moe-dense-y.f32"), np.float32).reshape(2, 4096)
    assert _sha(golden) == man["files"]["dense-y.f32"]["sha256"]
    gs = float(np.float32(man["synthetic"]["nvfp4_global_scale"]))
    g, u, d = s["dense"]
    y = orc.ffn(g, gs, u, gs, d, gs, 4096, 12288, s["x_dense"], limit=10.0, threads=8, path=1)
    for t in range(2):
        a, b = y[t].astype(np.float64), golden[t].astype(np.float64)
        cos = a @ b / np.sqrt((a @ a) * (b @ b))
        assert cos >= 0.9999  # the reference's gate (glm5_moe.rs:2531)
        assert 1 - cos < 1e-10 and np.max(np.abs(a - b)) < 2e-2  # what a correct f32 path actually reaches


# ---------------------------------------------------------------- router, argmax, combine

def test_router_matches_a_sort_based_brute_force():
    g = np.random.default_rng(11)
    for E, K, T in [(8, 2, 5), (64, 6, 7), (256, 8, 9), (512, 10, 3)]:
        logits = g.standard_normal((T, E)).astype(np.float32)
        ids, w = orc.router_topk(logits, K)
        p = np.exp(logits.astype(np.float64) - logits.max(1, keepdims=True))
        p /= p.sum(1, keepdims=True)
        order = np.argsort(-p, axis=1, kind="stable")[:, :K]
        assert np.array_equal(ids, order.astype(np.int32))
        wr = np.take_along_axis(p, order, 1)
        wr /= wr.sum(1, keepdims=True)
        assert np.allclose(w, wr, rtol=2e-6, atol=0)
        assert np.allclose(w.sum(1), 1.0, atol=1e-6)


def test_router_ties_go_to_the_lowest_index():
    logits = np.zeros((1, 16), np.float32)
    logits[0, [3, 9, 12]] = 2.0
    ids, w = orc.router_topk(logits, 4)
    assert ids.tolist() == [[3, 9, 12, 0]]
    assert np.allclose(w[0, :3], w[0, 0])


def test_argmax_rule():
    g = np.random.default_rng(3)
    for n in (1, 5, 1023, 1024, 1025, 151936):
        l = g.standard_normal(n).astype(np.float32)
        assert orc.argmax_ref(l) == int(np.argmax(l))
    # ties: the halving tree (strides 512 .. 1, left slot kept) prefers even slots in its last round,
    # then slots with bit 1 clear, ...: smallest bit-reversed (i mod 1024), then smallest i.
    l = np.zeros(4096, np.float32)
    l[[1030, 7, 2055]] = 5.0  # slots 6, 7, 7: 6 is even
    assert orc.argmax_ref(l) == 1030
    l = np.zeros(5, np.float32)
    l[[2, 4]] = 5.0  # by hand: stride 4 moves slot 4 into slot 0, stride 2 then keeps slot 0 -> index 4
    assert orc.argmax_ref(l) == 4
    l = np.zeros(2048, np.float32)
    l[[1, 1024 + 512, 512]] = 1.0  # slots 1, 512, 512: stride 512 pairs slot 0 with 512 -> slot 0 holds 512 (smallest i of the two)
    assert orc.argmax_ref(l) == 512
    l = np.full(3000, -3.2e38, np.float32)  # everything below the start value: index 0
    assert orc.argmax_ref(l) == 0


def test_acc_combo_and_silu_combo_small():
    g = np.random.default_rng(5)
    T, K, H, I = 3, 4, 8, 6
    x = g.standard_normal((T * K, H)).astype(np.float32)
    rw = g.random((T, K)).astype(np.float32)
    y0 = g.standard_normal((T, H)).astype(np.float32)
    y = orc.acc_combo(x, rw, T, K, H, y0)
    f = np.float32
    for t in range(T):
        for c in range(H):
            acc = f(0)
            for j in range(K):
                acc = f(acc + f(rw[t, j] * x[t * K + j, c]))
            assert y[t, c] == f(y0[t, c] + acc)
    h1 = g.standard_normal((5, 2 * I)).astype(np.float32)
    h2 = orc.silu_mul_combo(h1, I)
    want = h1[:, :I].astype(np.float64) / (1 + np.exp(-h1[:, :I].astype(np.float64))) * h1[:, I:]
    assert np.allclose(h2, want, rtol=1e-6, atol=1e-30)


def test_moe_layer_is_the_staged_composition():
    g = np.random.default_rng(9)
    E, H, I, K, T = 8, 128, 64, 2, 3
    from refgen import random_nvfp4
    gu = random_nvfp4(1, E * 2 * I, H)
    dn = random_nvfp4(2, E * H, I)
    x = g.standard_normal((T, H)).astype(np.float32)
    logits = g.standard_normal((T, E)).astype(np.float32)
    ids, w, y = orc.moe_layer(gu, 1e-3, dn, 2e-3, E, H, I, x, logits, K)
    ids2, w2 = orc.router_topk(logits, K)
    assert np.array_equal(ids, ids2) and np.array_equal(w, w2)
    gub, dnb = orc.byte_len(2 * I, H), orc.byte_len(H, I)
    want = np.zeros((T, H), np.float32)
    for t in range(T):
        acc = np.zeros(H, np.float32)
        for j in range(K):
            e = ids[t, j]
            h1 = orc.gemv(gu[e * gub:(e + 1) * gub], 2 * I, H, 1e-3, x[t])
            h2 = orc.silu_mul(h1[0, :I], h1[0, I:])
            eo = orc.gemv(dn[e * dnb:(e + 1) * dnb], H, I, 2e-3, h2)[0]
            acc = (acc + w[t, j] * eo).astype(np.float32)
        want[t] = acc
    assert np.array_equal(want.view(np.uint32), y.view(np.uint32))


def test_bf16_keep_gemv_is_the_exact_rational_dot_product():
    """gemv_bf16's f64 evaluation against exact rational arithmetic on small inputs (a transposed operand, a dropped
    column or a wrong widening of the bf16 bits would show)."""
    from fractions import Fraction
    rng = np.random.default_rng(5)
    rows, cols, t = 5, 24, 2
    w_bits = rng.integers(0, 1 << 16, size=(rows, cols), dtype=np.uint16)
    w_bits[(w_bits & 0x7F80) == 0x7F80] = 0x3F80  # no inf / nan
    w_bits = (w_bits & 0x8FFF) | 0x3000           # exponents near 1: no overflow in the exact sum
    x = rng.standard_normal((t, cols)).astype(np.float32)
    y = orc.gemv_bf16(w_bits, rows, cols, x)
    wf = orc.bf16_bits_to_f32(w_bits)
    assert np.array_equal(wf.view(np.uint32), w_bits.astype(np.uint32) << 16)
    for ti in range(t):
        for r in range(rows):
            exact = sum(Fraction(float(wf[r, k])) * Fraction(float(x[ti, k])) for k in range(cols))
            assert y[ti, r] == np.float32(float(exact)), (ti, r)


def test_f32_keep_gemv_is_the_exact_rational_dot_product_and_the_reference_order_agrees():
    """gemv_f32w's f64 evaluation against exact rational arithmetic on small inputs; the restatement of the reference's
    own order (256 strided partial sums, halving tree) against a plain loop written from kernels.rs:104-114, and within
    the f32 summation bound of the exact value."""
    from fractions import Fraction
    rng = np.random.default_rng(6)
    rows, cols, t = 4, 28, 2
    w = rng.standard_normal((rows, cols)).astype(np.float32)
    x = rng.standard_normal((t, cols)).astype(np.float32)
    y = orc.gemv_f32w(w, rows, cols, x)
    for ti in range(t):
        for r in range(rows):
            exact = sum(Fraction(float(w[r, k])) * Fraction(float(x[ti, k])) for k in range(cols))
            assert y[ti, r] == np.float32(float(exact)), (ti, r)
    # the reference's order, scalar loop: K = 600 leaves threads 88..255 with two terms and the rest with three
    rows, cols = 3, 600
    w = rng.standard_normal((rows, cols)).astype(np.float32)
    x = rng.standard_normal((1, cols)).astype(np.float32)
    got = orc.gemv_f32w_reference_order(w, rows, cols, x)
    for r in range(rows):
        red = [np.float32(0.0)] * 256
        for th in range(256):
            acc = np.float32(0.0)
            for i in range(th, cols, 256):
                acc = np.float32(acc + np.float32(w[r, i] * x[0, i]))
            red[th] = acc
        st = 128
        while st > 0:
            for th in range(st):
                red[th] = np.float32(red[th] + red[th + st])
            st >>= 1
        assert got[0, r] == red[0], r
    exact = orc.gemv_f32w(w, rows, cols, x).astype(np.float64)
    bound = orc.gamma(16 * (cols + 6)) * (np.abs(x.astype(np.float64)) @ np.abs(w.astype(np.float64)).T)
    assert np.all(np.abs(got.astype(np.float64) - exact) <= bound)
    # integers: every order gives the same exact sum
    wi = rng.integers(-8, 9, size=(5, 512)).astype(np.float32)
    xi = rng.integers(-8, 9, size=(2, 512)).astype(np.float32)
    assert np.array_equal(orc.gemv_f32w(wi, 5, 512, xi), orc.gemv_f32w_reference_order(wi, 5, 512, xi))
    assert np.array_equal(orc.gemv_f32w(wi, 5, 512, xi), (xi.astype(np.int64) @ wi.astype(np.int64).T).astype(np.float32))

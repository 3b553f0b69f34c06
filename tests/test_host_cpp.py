"""The C++ host layer (crow_nest_amd/host: the reference's Rust interface restated in C++ above the C ABI) through its
test driver tests/host_cpp/host_parity.  The driver holds no oracle: this file writes its inputs, runs it, and checks
what it hands back - on the CPU for the table, the container reader and the refusal texts, on the GPU for the engine's
callers (dense_ffn_w, dense_proj, lm_head_row, moe_run, gemm, load_fp4 from a container)."""
import json
import os
import struct
import subprocess

import numpy as np
import pytest

from conftest import GOLDEN, ROOT
from crow_nest_amd.cnq import Cnq, CnqRefused, sha256_hex
from oracle import oracle as orc
from refgen import normal_f32, random_nvfp4

EXE = os.path.join(ROOT, "tests", "host_cpp", "host_parity")
FIXTURE = os.path.join(GOLDEN, "synthetic-v2.cnq")


def _exe() -> str:
    if not os.path.exists(EXE):  # built by __graft_entry__.build(); g++ only, a few seconds
        for d in (os.path.join(ROOT, "crow_nest_amd", "host"), os.path.join(ROOT, "tests", "host_cpp")):
            r = subprocess.run(["make", "-C", d], capture_output=True, text=True)
            assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    return EXE


def run(*args, timeout=120) -> str:
    r = subprocess.run([_exe(), *[str(a) for a in args]], capture_output=True, text=True, timeout=timeout)
    assert r.returncode == 0, f"host_parity {args}: rc {r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-2000:]}"
    return r.stdout


# ---------------------------------------------------------------- CPU: table, types, container reader

def test_a_missing_kernel_panics_with_the_reference_text():
    assert run("missing").strip() == "kernel missing: gemv_nvfp4_nope"  # kernels.rs:5238


def test_nvfp4_matrix_checks_and_their_texts():
    out = run("matrix-checks").splitlines()  # cpu_nvfp4.rs:118-141
    assert out == ["cpu_nvfp4: 96 columns are not whole 64-value NVFP4 blocks", "cpu_nvfp4: [2, 128] needs 144 B, got 72", "ok 2 64 50135040"]


def test_expert_block_checks_and_their_texts():
    out = run("expert-checks").splitlines()  # cpu_nvfp4.rs:153-178
    gu, dn = 64 * 2 * 36, 128 * 36
    assert out == [f"cpu_nvfp4: expert unit H 128 I 64 needs {2 * gu + dn} B, got {2 * gu + dn - 1}",
                   "cpu_nvfp4: expert shapes gate [64, 128], up [64, 128], down [64, 128] do not fit together",
                   f"ok H 128 I 64 gate 0 up {gu} down {2 * gu} scales 1 2 3"]


def test_container_table_equals_the_python_reader():
    out = run("cnq-list", FIXTURE).splitlines()
    c = Cnq.open(FIXTURE)
    m = c.model()
    assert out[0] == (f"family={c.family()} model_type={m.model_type} recipe={m.recipe} repo={m.source_repo} revision={m.source_revision} "
                      f"blob_offset={c.blob_offset} tensors={len(c.tensors)}")
    assert len(out) == len(c.tensors) + 2
    for line, t in zip(out[1:], c.tensors):
        name, sec, dtype, off, n, blen, gs, shape = line.split("|")
        assert (name, sec, dtype, int(off), int(n), int(blen)) == (t.name, t.section, t.dtype, t.offset, t.n_values, Cnq.byte_len(t))
        assert np.float32(float(gs)) == np.float32(t.global_scale)
        assert tuple(int(v) for v in shape.split(",") if v) == tuple(t.shape)
    assert out[-1] == "find: tensor not found: lm_head.weight [no-such-section]"  # cnq.rs:1051-1062
    c.close()


def _container(tmp_path, index, name="t.cnq", magic=b"CNQ1", raw_index=None):
    ib = raw_index if raw_index is not None else json.dumps(index).encode()
    p = tmp_path / name
    p.write_bytes(magic + b"\0" * 8 + b"\0" * 64 + ib + struct.pack("<Q", len(ib)))
    return str(p)


def _v2(**over):
    cfg, gen = '{"model_type": "x"}', "{}"
    idx = {"format": "crow-nest-quant", "format_version": 2, "blob_offset": 12, "recipe": "r", "tensors": [],
           "model": {"family": "Qwen35Dense", "model_type": "x", "config_json": cfg, "config_json_sha256": sha256_hex(cfg.encode()),
                     "generation_config_json": gen, "generation_config_json_sha256": sha256_hex(gen.encode()),
                     "source": {"repo": "a/b", "revision": "r1", "shards": []}, "geo": {}}}
    idx.update(over)
    return idx


def test_refusals_equal_the_python_reader_and_so_the_reference(tmp_path):
    """Every refusal of open_checked (cnq.rs:143-239): the C++ text equals the Python reader's, which the reader's own
    tests hold to the reference's."""
    cases = []
    small = tmp_path / "small.cnq"
    small.write_bytes(b"CNQ1" + b"\0" * 10)
    cases.append(str(small))
    cases.append(_container(tmp_path, _v2(), name="magic.cnq", magic=b"CNQ2"))
    long_idx = tmp_path / "len.cnq"
    long_idx.write_bytes(b"CNQ1" + b"\0" * 40 + struct.pack("<Q", 1 << 40))
    cases.append(str(long_idx))
    cases.append(_container(tmp_path, _v2(format_version=3), name="fv3.cnq"))
    cases.append(_container(tmp_path, {"version": 1, "blob_offset": 12, "tensors": []}, name="v1.cnq"))
    cases.append(_container(tmp_path, {"version": 7, "blob_offset": 12}, name="v7.cnq"))
    altered = _v2()
    altered["model"]["config_json"] = '{"model_type": "y"}'
    cases.append(_container(tmp_path, altered, name="altered.cnq"))
    nomodel = _v2()
    del nomodel["model"]
    cases.append(_container(tmp_path, nomodel, name="nomodel.cnq"))
    nofam = _v2()
    del nofam["model"]["family"]
    cases.append(_container(tmp_path, nofam, name="nofam.cnq"))
    noblob = _v2()
    del noblob["blob_offset"]
    cases.append(_container(tmp_path, noblob, name="noblob.cnq"))
    for path in cases:
        with pytest.raises(CnqRefused) as ei:
            Cnq.open_checked(path)
        assert run("cnq-refuse", path).strip() == str(ei.value), path
    assert run("cnq-refuse", _container(tmp_path, _v2(), name="ok.cnq")).strip() == "accepted"
    assert run("cnq-refuse", FIXTURE).strip() == "accepted"
    # unicode and escapes in the stored config survive the index parser (the hash is over the decoded text)
    cfg = '{"model_type": "x", "note": "café \\"quoted\\" \U0001F426"}'
    uni = _v2()
    uni["model"]["config_json"] = cfg
    uni["model"]["config_json_sha256"] = sha256_hex(cfg.encode())
    assert run("cnq-refuse", _container(tmp_path, uni, name="uni.cnq")).strip() == "accepted"
    assert run("cnq-refuse", _container(tmp_path, None, name="uni2.cnq", raw_index=json.dumps(uni, ensure_ascii=False).encode())).strip() == "accepted"


# ---------------------------------------------------------------- GPU: the engine's callers

def _write(d, name, a):
    np.ascontiguousarray(a).tofile(os.path.join(d, name))


def _read(d, name, dtype, shape):
    return np.fromfile(os.path.join(d, name), dtype=dtype).reshape(shape)


def _bf16(x):
    bits = orc.f32_to_bf16_bits(x)
    return bits, orc.bf16_bits_to_f32(bits)


@pytest.mark.gpu
@pytest.mark.parametrize("t,xbf16", [(1, 0), (3, 0), (1, 1), (4, 1), (7, 0)])
def test_dense_ffn_w_and_dense_proj(tmp_path, t, xbf16):
    """dense_ffn_w for the decode / verify widths (gate_up + down, f32 and bf16 x), and dense_proj's three branches on f32 x:
    one row (gemv_nvfp4_w), 2..4 rows (gemv_nvfp4_wm), more (gemv_fp4_b)."""
    from gpu_common import TOL, rel_err
    H, I, R = 1024, 2816, 1024
    d = str(tmp_path)
    wg, wu, wd = random_nvfp4(41, I, H), random_nvfp4(42, I, H), random_nvfp4(43, R, I)
    gs = np.array([2.0e-3, 1.5e-3, 1.1e-3], np.float32)
    x = normal_f32(9, t, t * H).reshape(t, H) * np.float32(0.05)
    for name, a in (("gate.bin", wg), ("up.bin", wu), ("down.bin", wd), ("gs.bin", gs)):
        _write(d, name, a)
    if xbf16:
        bits, xw = _bf16(x)
        _write(d, "x.bin", bits)
        xw = xw.reshape(t, H)
    else:
        xw = x
        _write(d, "x.bin", x)
    open(os.path.join(d, "meta.txt"), "w").write(f"{H} {I} {R} {t} {xbf16}\n")
    run("dense", d)
    if t <= 4:
        h_ref = orc.silu_mul(orc.gemv(wg, I, H, gs[0], xw), orc.gemv(wu, I, H, gs[1], xw))
        assert rel_err(_read(d, "h.bin", np.float32, (t, I)), h_ref) <= TOL
        assert rel_err(_read(d, "y.bin", np.float32, (t, R)), orc.gemv(wd, R, I, gs[2], h_ref)) <= TOL
    if not xbf16:
        assert rel_err(_read(d, "gate_y.bin", np.float32, (t, I)), orc.gemv(wg, I, H, gs[0], xw)) <= TOL
    if t == 1 and not xbf16:  # the captured step, replayed three times: the eager launches' bits
        assert np.array_equal(_read(d, "y_graph.bin", np.uint32, (1, R)), _read(d, "y.bin", np.uint32, (1, R)))


@pytest.mark.gpu
def test_lm_head_row_returns_the_greedy_token(tmp_path):
    from gpu_common import TOL, rel_err
    V, K = 4000, 1024
    d = str(tmp_path)
    w = random_nvfp4(51, V, K)
    gs = np.array([1.0e-3], np.float32)
    x = normal_f32(10, 1, K)
    for name, a in (("w.bin", w), ("gs.bin", gs), ("x.bin", x)):
        _write(d, name, a)
    open(os.path.join(d, "meta.txt"), "w").write(f"{V} {K}\n")
    out = run("head", d)
    logits = _read(d, "logits.bin", np.float32, (V,))
    assert rel_err(logits, orc.gemv(w, V, K, gs[0], x)[0]) <= TOL
    assert int(out.split("token=")[1]) == orc.argmax_ref(logits)  # exact on the logits the device wrote


@pytest.mark.gpu
@pytest.mark.parametrize("t", [1, 4, 6])
def test_moe_run(tmp_path, t):
    from gpu_common import TOL, rel_err
    E, K, H, I = 64, 4, 512, 256  # the routing kernels take 64..1024 experts
    d = str(tmp_path)
    gu, dn = random_nvfp4(61, E * 2 * I, H), random_nvfp4(62, E * H, I)
    gs = np.array([1.3e-3, 0.9e-3], np.float32)
    x = normal_f32(11, 1, t * H).reshape(t, H) * np.float32(0.1)
    logits = normal_f32(12, 1, t * E).reshape(t, E)
    for name, a in (("gu.bin", gu), ("dn.bin", dn), ("gs.bin", gs), ("x.bin", x), ("logits.bin", logits)):
        _write(d, name, a)
    open(os.path.join(d, "meta.txt"), "w").write(f"{E} {K} {H} {I} {t}\n")
    run("moe", d)
    ids_ref, wts_ref, y_ref = orc.moe_layer(gu, gs[0], dn, gs[1], E, H, I, x, logits, K)
    assert np.array_equal(_read(d, "ids.bin", np.int32, (t, K)), np.asarray(ids_ref).reshape(t, K))
    assert np.allclose(_read(d, "wts.bin", np.float32, (t, K)), np.asarray(wts_ref).reshape(t, K), rtol=1e-6, atol=1e-7)
    assert rel_err(_read(d, "y.bin", np.float32, (t, H)), np.asarray(y_ref).reshape(t, H)) <= TOL


@pytest.mark.gpu
def test_moe_run_grouped(tmp_path):
    from gpu_common import TOL, rel_err
    E, K, H, I, t = 64, 4, 512, 256, 24
    d = str(tmp_path)
    gu, dn = random_nvfp4(63, E * 2 * I, H), random_nvfp4(64, E * H, I)
    gs = np.array([1.3e-3, 0.9e-3], np.float32)
    x = normal_f32(14, 1, t * H).reshape(t, H) * np.float32(0.1)
    logits = normal_f32(15, 1, t * E).reshape(t, E)
    for name, a in (("gu.bin", gu), ("dn.bin", dn), ("gs.bin", gs), ("x.bin", x), ("logits.bin", logits)):
        _write(d, name, a)
    open(os.path.join(d, "meta.txt"), "w").write(f"{E} {K} {H} {I} {t}\n")
    run("moe-grouped", d)
    ids_ref, wts_ref, y_ref = orc.moe_layer(gu, gs[0], dn, gs[1], E, H, I, x, logits, K, threads=4)
    assert np.array_equal(_read(d, "ids.bin", np.int32, (t, K)), np.asarray(ids_ref).reshape(t, K))
    assert rel_err(_read(d, "y.bin", np.float32, (t, H)), np.asarray(y_ref).reshape(t, H)) <= TOL


@pytest.mark.gpu
def test_keep_projections(tmp_path):
    from gpu_common import TOL, rel_err
    rows, k, t = 256, 2560, 2
    d = str(tmp_path)
    w = normal_f32(16, 1, rows * k).reshape(rows, k) * np.float32(0.05)
    bits = orc.f32_to_bf16_bits(w).reshape(rows, k)
    x = normal_f32(17, 1, t * k).reshape(t, k)
    for name, a in (("w_bf16.bin", bits), ("w_f32.bin", w), ("x.bin", x)):
        _write(d, name, a)
    open(os.path.join(d, "meta.txt"), "w").write(f"{rows} {k} {t}\n")
    run("keeps", d)
    assert rel_err(_read(d, "y_bf16.bin", np.float32, (t, rows)), orc.gemv_bf16(bits, rows, k, x)) <= TOL
    assert rel_err(_read(d, "y_f32.bin", np.float32, (t, rows)), orc.gemv_f32w(w, rows, k, x)) <= TOL


@pytest.mark.gpu
def test_gemm(tmp_path):
    from gpu_common import TOL, rel_err
    rows, cols, m = 320, 1024, 40
    d = str(tmp_path)
    w = random_nvfp4(71, rows, cols)
    gs = np.array([6.0e-4], np.float32)
    bits, xw = _bf16(normal_f32(13, 1, m * cols))
    for name, a in (("w.bin", w), ("gs.bin", gs), ("x.bin", bits)):
        _write(d, name, a)
    open(os.path.join(d, "meta.txt"), "w").write(f"{rows} {cols} {m}\n")
    run("gemm", d)
    assert rel_err(_read(d, "y.bin", np.float32, (m, rows)), orc.gemv(w, rows, cols, gs[0], xw.reshape(m, cols), threads=4)) <= TOL


@pytest.mark.gpu
def test_load_fp4_from_the_reference_container_dequantises_bit_exactly(tmp_path):
    d = str(tmp_path)
    out = run("cnq-dequant", FIXTURE, d)
    assert "load_fp4: model.language_model.layers.0.linear_attn.A_log: expected NVFP4, got f32" in out  # weights.rs:26-28
    c = Cnq.open(FIXTURE)
    seen = 0
    for i, t in enumerate(c.tensors):
        if t.dtype != "nvfp4" or len(t.shape) != 2:
            continue
        got = _read(d, f"{i}.f32", np.float32, t.shape)
        want = orc.dequant(c.read_bytes(t), t.global_scale).reshape(t.shape)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), t.name
        seen += 1
    assert seen == 6
    c.close()


@pytest.mark.gpu
def test_quantize_nvfp4_through_the_host_layer(tmp_path):
    """crow::quantize_nvfp4 (the converter's ceiling encoder, converter/src/main.rs:534-664): the blocks and the global scale
    of the CPU restatement byte for byte, and the converter's assert text for a ragged value count."""
    d = str(tmp_path)
    v = normal_f32(77, 4096, 4096 * 64) * np.float32(0.02)
    v[:64] = 0.0          # an all-zero block
    v[64] = 3.0           # the tensor's maximum: its sub-block takes the top scale byte
    _write(d, "values.bin", v)
    out = run("quantize", d)
    blocks, gs = orc.quantize_ceil(v)
    assert np.array_equal(_read(d, "blocks.bin", np.uint8, (-1,)), np.asarray(blocks).reshape(-1))
    assert _read(d, "gs.bin", np.float32, (1,))[0] == np.float32(gs)
    assert "ragged: assertion failed: values.len() % 64 == 0" in out


@pytest.mark.gpu
def test_panics_carry_the_reference_texts():
    out = run("panics").splitlines()
    assert out == ["f: kernel missing: gemv_nvfp4_nope", "proj_m: proj_m: M = 5 is outside 1..=4"]

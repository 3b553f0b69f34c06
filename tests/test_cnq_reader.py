"""The CNQ1 container reader against the reference's own container fixture (synthetic-v2.cnq, an index v2 written
by the reference's converter) and against its refusal texts (engine/src/cnq.rs:143-239, tests :1590-1700)."""
import json
import os
import struct

import numpy as np
import pytest

from conftest import GOLDEN
from crow_nest_amd.cnq import CNQ45M_INDEX_LEN, Cnq, CnqRefused, V1_REFUSAL, classify_index, sha256_hex
from oracle import oracle as orc
from refgen import lcg_bf16_tensors

FIXTURE = os.path.join(GOLDEN, "synthetic-v2.cnq")
NVFP4 = ["model.language_model.layers.0.linear_attn.in_proj_qkv.weight", "model.language_model.layers.0.linear_attn.out_proj.weight",
         "model.language_model.layers.0.mlp.gate_proj.weight", "model.language_model.layers.1.self_attn.q_proj.weight",
         "model.language_model.layers.1.mlp.down_proj.weight", "lm_head.weight"]


def test_opens_the_reference_fixture_as_index_v2():
    c = Cnq.open(FIXTURE)
    assert c.blob_offset == 12 and len(c.tensors) == 15
    m = c.model()
    assert m is not None and c.family() == "Qwen35Dense" and m.model_type == "qwen3_5_text" and m.recipe == "cnq4.5-qwen35-dense"
    assert m.source_repo == "crow-nest/synthetic-v2" and m.source_revision == "c6"
    assert json.loads(m.config_json)["model_type"].startswith("qwen3_5")
    assert [t.name for t in c.tensors if t.dtype == "nvfp4"] == NVFP4
    # byte_len per dtype, and the table is contiguous from the blob start
    at = 0
    raw_len = os.path.getsize(FIXTURE)
    for t in c.tensors:
        assert t.offset == at
        at += Cnq.byte_len(t)
    assert c.blob_offset + at <= raw_len - 8
    a = c.find("model.language_model.layers.0.linear_attn.A_log", "text")
    assert a.dtype == "f32" and Cnq.byte_len(a) == 8 and a.global_scale == 1.0
    assert Cnq.byte_len(c.find("mtp.fc.weight", "mtp")) == 16384
    with pytest.raises(KeyError, match=r"tensor not found: lm_head.weight \[mtp\]"):
        c.find("lm_head.weight", "mtp")  # always filter by section
    c.close()


def test_tensor_bytes_are_the_encoder_output_of_the_lcg_source():
    """read_bytes / read_range return exactly what the ceil encoder makes of the reference's LCG source tensors."""
    c = Cnq.open(FIXTURE)
    src = lcg_bf16_tensors()
    for name in NVFP4:
        t = c.find(name, "text")
        got = c.read_bytes(t)
        want, gs = orc.quantize_ceil(src[name])
        assert np.array_equal(got, want) and np.float32(gs) == np.float32(t.global_scale)
        rb = t.shape[1] // 64 * 36
        assert np.array_equal(c.read_range(t, 3 * rb, 2 * rb), want[3 * rb:5 * rb])  # rows 3..4
    with pytest.raises(CnqRefused):
        c.read_range(c.find("mtp.fc.weight", "mtp"), 16384, 1 << 20)
    c.close()


def _container(tmp_path, index: dict, payload: bytes = b"\0" * 64, name="t.cnq", magic=b"CNQ1"):
    ib = json.dumps(index).encode()
    p = tmp_path / name
    p.write_bytes(magic + b"\0" * 8 + payload + ib + struct.pack("<Q", len(ib)))
    return str(p), ib


def _v2(**over):
    cfg, gen = '{"model_type": "x"}', "{}"
    idx = {"format": "crow-nest-quant", "format_version": 2, "blob_offset": 12, "recipe": "r", "tensors": [],
           "model": {"family": "Qwen35Dense", "model_type": "x", "config_json": cfg, "config_json_sha256": sha256_hex(cfg.encode()),
                     "generation_config_json": gen, "generation_config_json_sha256": sha256_hex(gen.encode()),
                     "source": {"repo": "a/b", "revision": "r1", "shards": []}, "geo": {}}}
    idx.update(over)
    return idx


def test_refusals_carry_the_reference_texts(tmp_path):
    p = tmp_path / "small.cnq"
    p.write_bytes(b"CNQ1" + b"\0" * 10)
    with pytest.raises(CnqRefused, match=r"\[cnq\] refused: .*small.cnq: 14 B is too small to be a CNQ1 container"):
        Cnq.open(str(p))
    path, _ = _container(tmp_path, _v2(), magic=b"CNQ2")
    with pytest.raises(CnqRefused, match=r"magic is \[67, 78, 81, 50\], not CNQ1"):
        Cnq.open_checked(path)
    p = tmp_path / "len.cnq"
    p.write_bytes(b"CNQ1" + b"\0" * 40 + struct.pack("<Q", 1000))
    with pytest.raises(CnqRefused, match="index length 1000 does not fit a 52 B file"):
        Cnq.open_checked(str(p))
    p = tmp_path / "json.cnq"
    p.write_bytes(b"CNQ1" + b"\0" * 40 + b"{nope" + struct.pack("<Q", 5))
    with pytest.raises(CnqRefused, match="index json: "):
        Cnq.open_checked(str(p))
    # index v1 that is not the container of record
    path, ib = _container(tmp_path, {"format": "crow-nest-quant", "version": 1, "blob_offset": 12, "tensors": []}, name="v1.cnq")
    with pytest.raises(CnqRefused) as ei:
        Cnq.open_checked(path)
    assert V1_REFUSAL in str(ei.value) and sha256_hex(ib) in str(ei.value) and f"{CNQ45M_INDEX_LEN} B" in str(ei.value)
    # ... but the same trailer is accepted when its hash IS the one of record (the reference tests that path the same way)
    assert classify_index(ib, json.loads(ib), v1_of_record=sha256_hex(ib)) is None
    path, _ = _container(tmp_path, {"version": 3, "blob_offset": 12, "tensors": []}, name="v3.cnq")
    with pytest.raises(CnqRefused, match="CNQ index `version` 3 without a `format_version`"):
        Cnq.open_checked(path)
    path, _ = _container(tmp_path, _v2(format_version=3), name="fv3.cnq")
    with pytest.raises(CnqRefused, match="CNQ index format_version 3 is not one this engine reads"):
        Cnq.open_checked(path)
    idx = _v2()
    del idx["model"]
    path, _ = _container(tmp_path, idx, name="nomodel.cnq")
    with pytest.raises(CnqRefused, match="CNQ index v2 without a `model` block"):
        Cnq.open_checked(path)
    idx = _v2()
    idx["model"]["config_json"] = '{"model_type": "y"}'
    path, _ = _container(tmp_path, idx, name="altered.cnq")
    with pytest.raises(CnqRefused, match="the stored config was altered"):
        Cnq.open_checked(path)
    idx = _v2()
    del idx["model"]["family"]
    path, _ = _container(tmp_path, idx, name="nofamily.cnq")
    with pytest.raises(CnqRefused, match="`model.family` missing or not a string"):
        Cnq.open_checked(path)
    idx = _v2()
    del idx["blob_offset"]
    path, _ = _container(tmp_path, idx, name="noblob.cnq")
    with pytest.raises(CnqRefused, match="index has no blob_offset"):
        Cnq.open_checked(path)
    assert Cnq.open_checked(_container(tmp_path, _v2(), name="ok.cnq")[0]).tensors == []


def test_load_path_checks_dtype_and_shape_before_any_device_call():
    from crow_nest_amd.weights import nvfp4_matrix_of
    c = Cnq.open(FIXTURE)
    with pytest.raises(AssertionError, match="mtp.fc.weight: expected NVFP4, got bf16"):
        nvfp4_matrix_of(c, "mtp.fc.weight", "mtp")
    m = nvfp4_matrix_of(c, "model.language_model.layers.1.mlp.down_proj.weight", "text")
    assert (m.rows, m.cols, m.bytes.size) == (64, 128, 4608) and np.float32(m.global_scale) == np.float32(9.300595411332324e-05)
    c.close()

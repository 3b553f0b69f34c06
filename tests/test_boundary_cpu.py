"""CPU-side checks of the drop-in boundary: the shared library loads and exports exactly what
include/crow_hip.h declares, host-side types refuse bad shapes with the reference's messages, and
nothing computes without a GPU (no CPU fallback)."""
import os
import re

import numpy as np
import pytest

from conftest import ROOT
from crow_nest_amd import lib as L
from crow_nest_amd.weights import Nvfp4Matrix


def _declared(header="crow_hip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(crow_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    assert os.path.exists(L.library_path()), "libcrow_hip.so is not built: run __graft_entry__.build()"
    lib = L.lib()
    declared = _declared()
    assert declared, "no declarations found"
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/crow_hip.h but not exported"
    assert sorted(L.EXPORTS) == declared
    # the timing and tuning helpers of the benchmark and the tests live in a header of their own, outside the product ABI
    bench = _declared("crow_hip_bench.h")
    assert bench == sorted(L.BENCH_EXPORTS) and not set(bench) & set(declared)
    for name in bench:
        assert hasattr(lib, name), f"{name} is declared in include/crow_hip_bench.h but not exported"


def test_kernel_table_names_without_a_device():
    lib = L.lib()
    n = lib.crow_hip_function_count()
    names = [lib.crow_hip_function_name(i).decode() for i in range(n)]
    for want in ["gemv_nvfp4_w", "gemv_nvfp4_gu", "gemv_nvfp4_gu_bf16", "gemv_nvfp4_wm", "gemv_nvfp4_gum", "gemv_fp4", "gemv_fp4_b", "gemv_fp4_bs",
                 "gemv_fp4_b1k", "gemv_fp4_ptrb", "router_top10", "silu_mul_combo", "acc_combo", "argmax_k",
                 "dequant_fp4_flat", "gemv_nvfp4_w_argmax", "moe_gate_up_silu", "moe_down_combine", "moe_route_gate_up_silu", "moe_group", "moe_gate_up_silu_grouped", "moe_down_grouped", "gemm_nvfp4_bf16",
                 "gemm_nvfp4_bf16_m16", "gemm_nvfp4_bf16_m32", "gemm_nvfp4_bf16_m64", "gemv_bf16_w", "gemv_bf16", "gemv_bf16_b", "gemv_b", "gemv_bf16_ws", "gemv_bf16_bs"]:
        assert want in names, want
    import ctypes as C
    out = C.c_void_p()
    assert lib.crow_hip_get_function(b"no_such_kernel", C.byref(out)) == -2  # CROW_ERR_KERNEL_MISSING
    assert b"kernel missing" in lib.crow_hip_error_string(-2)
    assert lib.crow_hip_tiled_bytes(17408, 5120) == 17408 * 5120 // 64 * 36 == lib.crow_hip_container_bytes(17408, 5120)
    assert lib.crow_hip_tiled_bytes(1, 64) == 2304  # one padded group: 16 rows x 256 columns
    assert lib.crow_hip_tiled_bytes(151936, 5120) == lib.crow_hip_container_bytes(151936, 5120)


def test_kernel_header_is_the_library_table():
    """include/crow_kernels.h lists every kernel name with the number of values its launch takes: same set, same counts."""
    import ctypes as C
    text = open(os.path.join(ROOT, "include", "crow_kernels.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    listed = {m.group(1): int(m.group(2)) for m in re.finditer(r"^CROW_KERNEL\((\w+),\s*(\d+)\)", text, flags=re.M)}
    lib = L.lib()
    table = {}
    for i in range(lib.crow_hip_function_count()):
        name = lib.crow_hip_function_name(i)
        f = C.c_void_p()
        assert lib.crow_hip_get_function(name, C.byref(f)) == 0
        table[name.decode()] = lib.crow_hip_function_arg_count(f)
    assert listed == table


def test_gemm_kernel_choice_names_table_entries():
    lib = L.lib()
    n = lib.crow_hip_function_count()
    names = {lib.crow_hip_function_name(i).decode() for i in range(n)}
    picks = {m: lib.crow_hip_gemm_kernel(17408, m).decode() for m in (1, 16, 17, 96, 97, 128, 256, 512, 1024, 4096)}
    assert set(picks.values()) <= names
    assert picks[16] == "gemm_nvfp4_bf16_m16" and picks[17] == picks[96] == "gemm_nvfp4_bf16_m32"
    assert all(v != "gemm_nvfp4_bf16_m16" for m, v in picks.items() if m > 16)  # that entry point refuses m > 16


def test_launch_dims_depend_on_the_matrix_only():
    import ctypes as C
    lib = L.lib()
    d1, d4 = L.Dims(), L.Dims()
    assert lib.crow_hip_launch_dims(b"gemv_nvfp4_w", 17408, 5120, 1, C.byref(d1)) == 0
    assert lib.crow_hip_launch_dims(b"gemv_nvfp4_wm", 17408, 5120, 1, C.byref(d4)) == 0
    # verify rows == decode row, bit for bit: same split of K over waves and slices (it fixes the order of the sums); the verify
    # kernel's blocks take two strips each, and the row hint differs
    assert (d1.gy & 0xFF0FFFFF, d1.gz, d1.bx) == (d4.gy & 0xFF0FFFFF, d4.gz, d4.bx) and d4.gx == (d1.gx + 1) // 2
    assert d1.gx == 17408 // 16 and d1.bx == 3 * 64 and d1.gy == (5120 // 64) | (1 << 24)  # one block per strip, whole K inside it
    assert (d4.gy >> 20) & 0xF == 1
    assert lib.crow_hip_launch_dims(b"gemv_nvfp4_w", 5120, 17408, 1, C.byref(d1)) == 0
    assert d1.gy >> 24 > 1 and d1.gy & 0xFFFFF == 17408 // 64  # a strip of 68 groups is cut into slices
    assert lib.crow_hip_launch_dims(b"gemv_nvfp4_gu_bf16", 17408, 5120, 1, C.byref(d1)) == 0
    assert d1.bx == 2 * 2 * 64 and d1.gy >> 24 == 1
    assert lib.crow_hip_launch_dims(b"gemv_nvfp4_w", 8, 96, 1, C.byref(d1)) == -7  # 96 columns: not whole blocks


def test_matrix_shapes_are_checked_like_the_reference():
    b = np.zeros(Nvfp4Matrix.byte_len(3, 128), np.uint8)
    Nvfp4Matrix.new(b, 3, 128, 1.0)
    with pytest.raises(ValueError, match="96 columns are not whole 64-value NVFP4 blocks"):
        Nvfp4Matrix.new(b, 3, 96, 1.0)
    with pytest.raises(ValueError, match=r"\[3, 128\] needs 216 B, got 215"):
        Nvfp4Matrix.new(b[1:], 3, 128, 1.0)


def test_expert_block_is_cut_out_of_a_unit_like_the_reference():
    """ExpertBlock::new / from_unit (engine/src/cpu_nvfp4.rs:153-178): gate | up | down back to back, the three global scales
    in that order, the reference's refusal texts."""
    from crow_nest_amd.weights import ExpertBlock
    hidden, inter = 128, 64
    gu, dn = Nvfp4Matrix.byte_len(inter, hidden), Nvfp4Matrix.byte_len(hidden, inter)
    unit = (np.arange(2 * gu + dn) % 251).astype(np.uint8)
    e = ExpertBlock.from_unit(unit, hidden, inter, (1.0, 2.0, 3.0))
    assert (e.hidden, e.inter) == (hidden, inter)
    assert np.array_equal(e.gate.bytes, unit[:gu]) and np.array_equal(e.up.bytes, unit[gu:2 * gu]) and np.array_equal(e.down.bytes, unit[2 * gu:])
    assert (e.gate.global_scale, e.up.global_scale, e.down.global_scale) == (1.0, 2.0, 3.0)
    assert (e.down.rows, e.down.cols) == (hidden, inter)
    with pytest.raises(ValueError, match=f"expert unit H 128 I 64 needs {2 * gu + dn} B, got {2 * gu + dn - 1}"):
        ExpertBlock.from_unit(unit[1:], hidden, inter, (1.0, 2.0, 3.0))
    with pytest.raises(ValueError, match=r"expert shapes gate \[64, 128\], up \[64, 128\], down \[64, 128\] do not fit together"):
        ExpertBlock.new(e.gate, e.up, e.gate)


def test_no_cpu_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    from crow_nest_amd.weights import load_fp4
    m = Nvfp4Matrix.new(np.zeros(Nvfp4Matrix.byte_len(64, 256), np.uint8), 64, 256, 1.0)
    with pytest.raises(RuntimeError, match="no HIP device"):
        load_fp4(m)


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "crow_nest_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".h", ".hip", ".cpp", "Makefile")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), (dirpath, f)


def test_group_layout_is_a_bijection_and_matches_the_matrix_operand_shape():
    """Every byte of a 2304-byte group (16 rows x 256 columns) is owned by exactly one (row, column) item, and the placement is
    the one the kernels assume: a lane's dword d of code half h is strip row lane % 16, pair 2 h + d / 2, segment d % 2, columns
    8 (lane / 16) .. + 7 of that segment; a lane's scale byte jj is row lane % 16, pair jj, segment g & 1, half g >> 1."""
    lib = L.lib()
    seen = set()
    for row in range(16):
        for wp in range(32):
            o = lib.crow_hip_tile_code_offset(row, wp)
            pair, seg, g = wp >> 3, (wp >> 2) & 1, wp & 3
            lane, h, d = 16 * g + row, pair >> 1, 2 * (pair & 1) + seg
            assert o == 256 + 1024 * h + 16 * lane + 4 * d and o % 4 == 0
            for b in range(4):
                assert o + b not in seen
                seen.add(o + b)
        for sb in range(16):
            o = lib.crow_hip_tile_scale_offset(row, sb)
            pair, seg, half = sb >> 2, (sb >> 1) & 1, sb & 1
            g = 2 * half + seg
            assert o == 4 * (16 * g + row) + pair and o < 256
            assert o not in seen
            seen.add(o)
    assert seen == set(range(2304))
    assert lib.crow_hip_tile_code_offset(16, 0) == 0xFFFFFFFF and lib.crow_hip_tile_scale_offset(0, 16) == 0xFFFFFFFF

"""Host-side weight types and the load path: container bytes -> device -> tiled layout.

Mirrors, for the NVFP4 path only:
  * ``cpu_nvfp4::Nvfp4Matrix`` (engine/src/cpu_nvfp4.rs:107-141): borrowed container bytes +
    rows / cols / global scale, with the same shape checks and error texts;
  * ``weights::load_fp4 -> Fp4 {w, gs}`` and ``PW::Fp4(w, gs)`` (engine/src/weights.rs:26-33,
    engine/src/gen.rs:234-237): device bytes + a one-float device scalar;
  * ``cpu_nvfp4::ExpertBlock`` with ``new`` and ``from_unit`` (engine/src/cpu_nvfp4.rs:143-179): one routed expert as three
    matrices, or cut out of a gate | up | down unit, same checks and texts;
  * the loader's scale rule 0x7F -> 0x7E (engine/src/gen.rs:2178-2187, residency.rs:126-137), which the
    library's repacker applies while it re-tiles (``crow_hip_repack_nvfp4``);
  * ``Params`` (engine/src/gen.rs:2913-2925): the 4-byte device words kernels read their scalars from.
  * ``load_fp4(cnq, name, sec)`` from an open container (``crow_nest_amd/cnq.py``): ``load_fp4_cnq``.
PyTorch tensors are used as device allocations only.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from . import lib as _l

BLOCK_BYTES = 36
BLOCK_VALUES = 64


@dataclass(frozen=True)
class Nvfp4Matrix:
    """One NVFP4 matrix [rows, cols] over container bytes on the host."""
    bytes: np.ndarray
    rows: int
    cols: int
    global_scale: float

    @staticmethod
    def byte_len(rows: int, cols: int) -> int:
        return rows * (cols // BLOCK_VALUES) * BLOCK_BYTES

    @staticmethod
    def new(data, rows: int, cols: int, global_scale: float) -> "Nvfp4Matrix":
        b = np.ascontiguousarray(np.asarray(data, dtype=np.uint8).reshape(-1))
        if cols == 0 or cols % BLOCK_VALUES != 0:
            raise ValueError(f"cpu_nvfp4: {cols} columns are not whole 64-value NVFP4 blocks")
        want = Nvfp4Matrix.byte_len(rows, cols)
        if b.size != want:
            raise ValueError(f"cpu_nvfp4: [{rows}, {cols}] needs {want} B, got {b.size}")
        return Nvfp4Matrix(b, rows, cols, float(np.float32(global_scale)))


@dataclass(frozen=True)
class ExpertBlock:
    """One routed expert on the host (``cpu_nvfp4::ExpertBlock``, engine/src/cpu_nvfp4.rs:143-179): gate [inter, hidden],
    up [inter, hidden], down [hidden, inter], each with its own global scale."""
    gate: Nvfp4Matrix
    up: Nvfp4Matrix
    down: Nvfp4Matrix
    hidden: int
    inter: int

    @staticmethod
    def new(gate: Nvfp4Matrix, up: Nvfp4Matrix, down: Nvfp4Matrix) -> "ExpertBlock":
        inter, hidden = gate.rows, gate.cols
        if (up.rows, up.cols) != (inter, hidden) or (down.rows, down.cols) != (hidden, inter):
            raise ValueError(f"cpu_nvfp4: expert shapes gate [{gate.rows}, {gate.cols}], up [{up.rows}, {up.cols}], "
                             f"down [{down.rows}, {down.cols}] do not fit together")
        return ExpertBlock(gate, up, down, hidden, inter)

    @staticmethod
    def from_unit(unit, hidden: int, inter: int, global_scales) -> "ExpertBlock":
        """One expert unit as the GLM converter writes it: gate | up | down back to back, global scales in that order
        (``ExpertBlock::from_unit``, engine/src/cpu_nvfp4.rs:165-178)."""
        b = np.ascontiguousarray(np.asarray(unit, dtype=np.uint8).reshape(-1))
        gu, dn = Nvfp4Matrix.byte_len(inter, hidden), Nvfp4Matrix.byte_len(hidden, inter)
        if b.size != 2 * gu + dn:
            raise ValueError(f"cpu_nvfp4: expert unit H {hidden} I {inter} needs {2 * gu + dn} B, got {b.size}")
        g0, g1, g2 = global_scales
        return ExpertBlock.new(Nvfp4Matrix.new(b[:gu], inter, hidden, g0), Nvfp4Matrix.new(b[gu:2 * gu], inter, hidden, g1),
                               Nvfp4Matrix.new(b[2 * gu:], hidden, inter, g2))


def load_expert_block(e: ExpertBlock):
    """The three matrices of one expert unit on the device, as an ``engine.MlpW`` (gate, up, down): the dense kernels
    (gemv_nvfp4_gu + gemv_nvfp4_w) then run the expert's FFN, each matrix under its own global scale."""
    from .engine import MlpW
    return MlpW(load_fp4(e.gate), load_fp4(e.up), load_fp4(e.down))


def _device() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("crow_nest_amd needs a gfx950 GPU: no HIP device is visible (there is no CPU path)")
    return torch.device("cuda", 0)


def tiled_bytes(rows: int, cols: int) -> int:
    return int(_l.lib().crow_hip_tiled_bytes(rows, cols))


@dataclass
class Fp4:
    """``PW::Fp4(w, gs)``: tiled weight bytes and the global scale, both on the device."""
    w: torch.Tensor   # uint8 [tiled_bytes]
    gs: torch.Tensor  # float32 [1]
    rows: int
    cols: int

    @property
    def w_ptr(self) -> int:
        return self.w.data_ptr()

    @property
    def gs_ptr(self) -> int:
        return self.gs.data_ptr()


def repack_into(raw_dev: torch.Tensor, rows: int, cols: int, dst: torch.Tensor) -> None:
    """Container bytes on the device -> tiled layout (applies the scale rule)."""
    _l.ensure_init()
    assert raw_dev.is_cuda and dst.is_cuda and raw_dev.dtype == torch.uint8 and dst.dtype == torch.uint8
    if raw_dev.numel() != Nvfp4Matrix.byte_len(rows, cols):
        raise ValueError(f"cpu_nvfp4: [{rows}, {cols}] needs {Nvfp4Matrix.byte_len(rows, cols)} B, got {raw_dev.numel()}")
    if dst.numel() < tiled_bytes(rows, cols):
        raise ValueError("tiled destination too small")
    _l.check(_l.lib().crow_hip_repack_nvfp4(raw_dev.data_ptr(), rows, cols, dst.data_ptr()), "crow_hip_repack_nvfp4")


def load_fp4(m: Nvfp4Matrix) -> Fp4:
    """``load_fp4``: upload the container bytes, re-tile them on the device, keep (w, gs)."""
    dev = _device()
    _l.ensure_init()
    raw = torch.from_numpy(m.bytes).to(dev)
    w = torch.empty(tiled_bytes(m.rows, m.cols), dtype=torch.uint8, device=dev)
    repack_into(raw, m.rows, m.cols, w)
    gs = torch.tensor([m.global_scale], dtype=torch.float32, device=dev)
    return Fp4(w, gs, m.rows, m.cols)


def nvfp4_matrix_of(cnq, name: str, sec: str) -> Nvfp4Matrix:
    """The container bytes of one 2-D NVFP4 tensor of an open CNQ1 container as an ``Nvfp4Matrix`` (host side).
    The dtype check and its text are ``weights::load_fp4``'s (engine/src/weights.rs:26-28); rows and cols come from the
    index entry's shape, and the byte length is checked against it as ``Nvfp4Matrix::new`` does."""
    t = cnq.find(name, sec)
    if t.dtype in ("bf16", "f32"):
        raise AssertionError(f"{name}: expected NVFP4, got {t.dtype}")
    if len(t.shape) != 2 or t.shape[0] * t.shape[1] != t.n_values:
        raise ValueError(f"{name}: shape {list(t.shape)} is not a matrix of {t.n_values} values")
    return Nvfp4Matrix.new(cnq.read_bytes(t), t.shape[0], t.shape[1], t.global_scale)


def load_fp4_cnq(cnq, name: str, sec: str) -> Fp4:
    """``weights::load_fp4(cnq, name, sec)`` (engine/src/weights.rs:26-33): read the tensor's bytes from the container,
    upload, re-tile on the device (the scale rule is applied there), keep (w, gs)."""
    return load_fp4(nvfp4_matrix_of(cnq, name, sec))


def load_expert_slabs_cnq(cnq, name: str, sec: str) -> ExpertSlabs:
    """An expert tensor [E][rows][cols] of a container, read slab by slab with ``read_range`` (row-aligned reads, as
    engine/src/residency.rs:108-117 cuts them) and re-tiled per expert."""
    t = cnq.find(name, sec)
    if t.dtype in ("bf16", "f32"):
        raise AssertionError(f"{name}: expected NVFP4, got {t.dtype}")
    if len(t.shape) != 3 or t.shape[0] * t.shape[1] * t.shape[2] != t.n_values:
        raise ValueError(f"{name}: shape {list(t.shape)} is not [experts][rows][cols] of {t.n_values} values")
    e, rows, cols = t.shape
    per = Nvfp4Matrix.byte_len(rows, cols)
    data = np.concatenate([cnq.read_range(t, i * per, per) for i in range(e)])
    return load_expert_slabs(data, e, rows, cols, t.global_scale)


def quantize_nvfp4(values: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``quantize_nvfp4`` with ceiling scales (converter/src/main.rs:550-664, ScalesMode::Ceil) on the device:
    f32 values (a multiple of 64; sub-blocks are 16 consecutive values) -> (container blocks, uint8 [n / 64 * 36]; the
    tensor's global scale, float32 [1]), byte for byte what the converter writes."""
    _l.ensure_init()
    v = values.reshape(-1)
    if not (v.is_cuda and v.dtype == torch.float32 and v.is_contiguous()):
        raise ValueError("quantize_nvfp4: f32 values on the device, contiguous")
    if v.numel() == 0 or v.numel() % BLOCK_VALUES != 0:
        raise ValueError(f"quantize_nvfp4: {v.numel()} values are not whole 64-value NVFP4 blocks")
    blocks = torch.empty(v.numel() // BLOCK_VALUES * BLOCK_BYTES, dtype=torch.uint8, device=v.device)
    gs = torch.empty(1, dtype=torch.float32, device=v.device)
    _l.check(_l.lib().crow_hip_quantize_nvfp4(v.data_ptr(), v.numel(), blocks.data_ptr(), gs.data_ptr()), "crow_hip_quantize_nvfp4")
    return blocks, gs


def load_fp4_quantized(blocks: torch.Tensor, gs: torch.Tensor, rows: int, cols: int) -> Fp4:
    """Container blocks already on the device (``quantize_nvfp4``'s) -> the tiled tensor the kernels read."""
    w = torch.empty(tiled_bytes(rows, cols), dtype=torch.uint8, device=blocks.device)
    repack_into(blocks, rows, cols, w)
    return Fp4(w, gs, rows, cols)


def unpack(w: Fp4) -> np.ndarray:
    """Tiled -> container bytes (scale bytes canonical); for round-trip checks."""
    out = torch.empty(Nvfp4Matrix.byte_len(w.rows, w.cols), dtype=torch.uint8, device=w.w.device)
    _l.check(_l.lib().crow_hip_unpack_nvfp4(w.w.data_ptr(), w.rows, w.cols, out.data_ptr()), "crow_hip_unpack_nvfp4")
    return out.cpu().numpy()


def dequant(w: Fp4) -> torch.Tensor:
    """f32 [rows, cols] on the device, bit-exact with the reference decode after the scale rule."""
    out = torch.empty((w.rows, w.cols), dtype=torch.float32, device=w.w.device)
    _l.check(_l.lib().crow_hip_dequant_tiled(w.w.data_ptr(), w.gs.data_ptr(), w.rows, w.cols, out.data_ptr()),
             "crow_hip_dequant_tiled")
    return out


@dataclass
class ExpertSlabs:
    """An expert tensor [E][rows][cols] re-tiled per expert: slab e starts at e * slab_bytes."""
    w: torch.Tensor
    gs: torch.Tensor
    experts: int
    rows: int
    cols: int
    slab_bytes: int

    def ptr(self, e: int) -> int:
        return self.w.data_ptr() + e * self.slab_bytes


def load_expert_slabs(data, experts: int, rows: int, cols: int, global_scale: float) -> ExpertSlabs:
    """Flash-Next style expert tensor (engine/src/residency.rs:108-117: one global scale, expert e's
    container slab at e * rows * cols / 64 * 36) -> per-expert contiguous tiled slabs."""
    dev = _device()
    _l.ensure_init()
    b = np.ascontiguousarray(np.asarray(data, dtype=np.uint8).reshape(-1))
    per = Nvfp4Matrix.byte_len(rows, cols)
    if b.size != experts * per:
        raise ValueError(f"cpu_nvfp4: [{experts}][{rows}, {cols}] needs {experts * per} B, got {b.size}")
    slab = tiled_bytes(rows, cols)
    raw = torch.from_numpy(b).to(dev)
    w = torch.empty(experts * slab, dtype=torch.uint8, device=dev)
    for e in range(experts):
        repack_into(raw[e * per:(e + 1) * per], rows, cols, w[e * slab:(e + 1) * slab])
    gs = torch.tensor([float(np.float32(global_scale))], dtype=torch.float32, device=dev)
    return ExpertSlabs(w, gs, experts, rows, cols, slab)


class Params:
    """Device words for kernel scalars (``Params`` of engine/src/gen.rs:2913-2925), created on demand."""

    def __init__(self):
        self._dev = _device()
        self._cache: dict[int, torch.Tensor] = {}

    def i32(self, v: int) -> int:
        t = self._cache.get(v)
        if t is None:
            t = torch.tensor([v], dtype=torch.int32, device=self._dev)
            self._cache[v] = t
        return t.data_ptr()

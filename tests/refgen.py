"""Deterministic generators used by the tests.

Two of them re-create inputs the reference's own tests generate (so that the fixtures the
reference holds can be checked without importing any of its code):

* ``SplitMix64``  - the PRNG of engine/src/cpu_nvfp4.rs:434-451 (also cpu_mul1.rs:2477-2490);
  counter based, so whole streams vectorise: state_k = seed + k * 0x9E3779B97F4A7C15.
* ``lcg_bf16_tensors`` - the LCG source of converter/src/main.rs:2552-2594 behind
  engine/tests/fixtures/synthetic-v2/synthetic-v2.cnq.

The third, ``normal_f32``, defines this repository's own seeded N(0, sigma^2) stream for the
benchmark configurations (the reference fixes no generator for them).
"""
from __future__ import annotations

import numpy as np

_G = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z: np.ndarray) -> np.ndarray:
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


class SplitMix64:
    """Vectorised splitmix64 with the reference's draw helpers."""

    def __init__(self, seed: int):
        self.seed = np.uint64(seed & 0xFFFFFFFFFFFFFFFF)
        self.k = 0  # draws made so far

    def next(self, n: int) -> np.ndarray:
        with np.errstate(over="ignore"):
            idx = np.arange(self.k + 1, self.k + n + 1, dtype=np.uint64)
            out = _mix(self.seed + idx * _G)
        self.k += n
        return out

    def skip(self, n: int) -> None:
        self.k += n

    def bytes(self, n: int) -> np.ndarray:
        return (self.next(n) & np.uint64(0xFF)).astype(np.uint8)

    def f(self, n: int, a: float) -> np.ndarray:
        """uniform in [-a, a): ((next >> 40) as f32 / 2^24 * 2 - 1) * a, every step in f32"""
        v = (self.next(n) >> np.uint64(40)).astype(np.float32)
        v = v / np.float32(16777216.0)
        v = v * np.float32(2.0) - np.float32(1.0)
        return (v * np.float32(a)).astype(np.float32)


def lcg_u32(seed: int, n: int) -> np.ndarray:
    """x_{k+1} = x_k * 1664525 + 1013904223 mod 2^32, the n values after ``seed``."""
    # closed form per index is awkward; a python loop over <1e6 values is fine for the fixture
    out = np.empty(n, np.uint32)
    x = seed & 0xFFFFFFFF
    for i in range(n):
        x = (x * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = x
    return out


SYNTHETIC_V2_TENSORS = [
    ("model.language_model.embed_tokens.weight", (128, 64)),
    ("model.language_model.layers.0.input_layernorm.weight", (64,)),
    ("model.language_model.layers.0.linear_attn.A_log", (2,)),
    ("model.language_model.layers.0.linear_attn.dt_bias", (2,)),
    ("model.language_model.layers.0.linear_attn.conv1d.weight", (128, 1, 4)),
    ("model.language_model.layers.0.linear_attn.in_proj_a.weight", (2, 64)),
    ("model.language_model.layers.0.linear_attn.in_proj_qkv.weight", (128, 64)),
    ("model.language_model.layers.0.linear_attn.out_proj.weight", (64, 64)),
    ("model.language_model.layers.0.mlp.gate_proj.weight", (128, 64)),
    ("model.language_model.layers.1.self_attn.q_proj.weight", (128, 64)),
    ("model.language_model.layers.1.self_attn.k_norm.weight", (32,)),
    ("model.language_model.layers.1.mlp.down_proj.weight", (64, 128)),
    ("model.language_model.norm.weight", (64,)),
    ("lm_head.weight", (128, 64)),
    ("mtp.fc.weight", (64, 128)),
    ("model.visual.blocks.0.attn.qkv.weight", (192, 64)),
]


def lcg_bf16_tensors() -> dict[str, np.ndarray]:
    """The BF16 source of synthetic-v2.cnq, widened to f32 (name -> flat f32 array)."""
    total = sum(int(np.prod(s)) for _, s in SYNTHETIC_V2_TENSORS)
    x = lcg_u32(0xC6C60300, total)
    v = (((x >> np.uint32(8)) % np.uint32(2001)).astype(np.float32) - np.float32(1000.0)) / np.float32(4000.0)
    bits = v.view(np.uint32) & np.uint32(0xFFFF0000)  # truncation to bf16, as the reference writes it
    vals = bits.view(np.float32)
    out, at = {}, 0
    for name, shape in SYNTHETIC_V2_TENSORS:
        n = int(np.prod(shape))
        out[name] = vals[at:at + n].copy()
        at += n
    return out


def normal_f32(seed: int, stream: int, n: int, sigma: float = 1.0) -> np.ndarray:
    """This repository's seeded N(0, sigma^2) f32 stream: splitmix64(seed * 2^32 + stream) uniforms
    through Box-Muller (pairs of draws; cos branch first, then sin), computed in f64, rounded to f32."""
    rng = SplitMix64(((seed & 0xFFFFFFFF) << 32) | (stream & 0xFFFFFFFF))
    m = (n + 1) // 2
    out = np.empty(2 * m, np.float32)
    step = 1 << 22
    for i in range(0, m, step):
        k = min(step, m - i)
        u = rng.next(2 * k)
        u1 = ((u[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) / 9007199254740993.0  # (0, 1)
        u2 = (u[1::2] >> np.uint64(11)).astype(np.float64) / 9007199254740992.0  # [0, 1)
        r = np.sqrt(-2.0 * np.log(u1)) * sigma
        out[2 * i:2 * (i + k):2] = (r * np.cos(2.0 * np.pi * u2)).astype(np.float32)
        out[2 * i + 1:2 * (i + k):2] = (r * np.sin(2.0 * np.pi * u2)).astype(np.float32)
    return out[:n]


def synth_nvfp4(rng: SplitMix64, rows: int, cols: int, scale_fn, code_mask: int = 0xFF) -> np.ndarray:
    """The reference tests' synthetic matrix (cpu_nvfp4.rs:454-465): per 36-byte block, 4 scale
    bytes from ``scale_fn(rng)`` (called once per byte, in order), then 32 code bytes."""
    nb = rows * cols // 64
    out = np.empty((nb, 36), np.uint8)
    for b in range(nb):
        for i in range(4):
            out[b, i] = scale_fn(rng)
        out[b, 4:] = rng.bytes(32) & code_mask
    return out.reshape(-1)


def scale_mix(rng: SplitMix64) -> int:
    """cpu_nvfp4.rs:467-475: 0x30..0x7F, about 1 in 16 is 0x7F"""
    b = int(rng.bytes(1)[0])
    return 0x7F if (b & 15) == 0 else 0x30 + (b >> 4) * 3


def random_nvfp4(seed: int, rows: int, cols: int, scale_lo: int = 0x28, scale_hi: int = 0x7F,
                 p7f: float = 1 / 64) -> np.ndarray:
    """Fast vectorised random NVFP4 bytes (this repository's own; not a reference stream)."""
    g = np.random.default_rng(seed)
    nb = rows * cols // 64
    out = g.integers(0, 256, size=(nb, 36), dtype=np.uint8)
    sc = g.integers(scale_lo, scale_hi, size=(nb, 4), dtype=np.uint8)
    if p7f > 0:
        sc[g.random((nb, 4)) < p7f] = 0x7F
    out[:, :4] = sc
    return out.reshape(-1)

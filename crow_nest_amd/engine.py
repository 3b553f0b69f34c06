"""The callers of the hot path, mirrored from the reference engine (engine/src/gen.rs).

Only the NVFP4 weight x activation dispatch is here - the functions a maintainer would touch to
put the HIP library behind ``gen.rs``:

    dense_proj    gen.rs:3915-3932   t == 1 -> gemv_nvfp4_w; 2..4 (verify) -> gemv_nvfp4_wm; more -> GEMM
    dense_ffn_w   gen.rs:3974-3992   t == 1 -> gemv_nvfp4_gu + down
    proj_m        gen.rs:5455-5466   gemv_nvfp4_wm over M <= 4 rows
    verify_ffn    gen.rs:5632-5634   gemv_nvfp4_gum + proj_m(down)
    lm_head_row   gen.rs:4766-4784   lm_head through dense_proj, then argmax_k (gen.rs:6197-6198)
    moe_run       gen.rs:4168-4534   router_top10 -> routed gate|up -> SwiGLU -> routed down -> acc_combo
Buffers are torch tensors on the device (allocation only); every launch goes through
``launch_v(k.f(name), ...)`` with device addresses, exactly like the reference call sites.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .kernels import KernelGeo, Kernels, compile, launch_dims, launch_v, set_geo, status
from .weights import ExpertSlabs, Fp4, Params

NVFP4_MMAX = 4  # kernels_p2.rs:397


@dataclass
class MlpW:
    gate: Fp4
    up: Fp4
    down: Fp4


@dataclass
class MoeW:
    gate_up: ExpertSlabs  # [E][2 I][H], gate rows 0..I, up rows I..2I
    down: ExpertSlabs     # [E][H][I]
    table: torch.Tensor   # u64 [E][2]: device address of expert e's gate_up / down slab (residency.rs table)


def expert_table(gate_up: ExpertSlabs, down: ExpertSlabs) -> torch.Tensor:
    rows = [[gate_up.ptr(e), down.ptr(e)] for e in range(gate_up.experts)]
    # addresses exceed int64's positive range never (48-bit), so int64 storage is exact
    return torch.tensor(rows, dtype=torch.int64, device=gate_up.w.device)


class Engine:
    def __init__(self, geo: KernelGeo | None = None):
        self.module = compile(geo)
        self.k = Kernels(self.module)
        self.p = Params()
        self.geo = geo or KernelGeo()
        self.dev = torch.device("cuda", 0)

    def set_geo(self, geo: KernelGeo) -> None:
        self.geo = geo
        set_geo(geo)

    def check(self) -> None:
        status()

    # ------------------------------------------------------------------ dense projections
    def dense_proj(self, w: Fp4, t: int, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        """y[t][rows] = x[t][cols] W^T.  x f32 or bf16 (bf16 only for t <= 4 and the GEMM)."""
        rows, k = w.rows, w.cols
        assert x.is_cuda and x.is_contiguous() and x.numel() == t * k
        if y is None:
            y = torch.empty((t, rows), dtype=torch.float32, device=self.dev)
        p = self.p
        if t == 1 and x.dtype == torch.float32:
            gx, gy, gz, bx = launch_dims("gemv_nvfp4_w", rows, k)
            launch_v(self.k.f("gemv_nvfp4_w"), gx, gy, gz, bx, [w.w_ptr, x.data_ptr(), w.gs_ptr, y.data_ptr(), p.i32(k), p.i32(rows)])
        elif t <= NVFP4_MMAX:
            self.proj_m(w, t, x, y)
        elif x.dtype == torch.bfloat16:
            self.gemm(w, t, x, y)
        else:
            gx, gy, gz, bx = launch_dims("gemv_fp4_b", rows, k, t)
            launch_v(self.k.f("gemv_fp4_b"), gx, gy, gz, bx,
                     [w.w_ptr, x.data_ptr(), w.gs_ptr, y.data_ptr(), p.i32(k), p.i32(rows), p.i32(t)])
        return y

    def proj_m(self, w: Fp4, m: int, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        rows, k = w.rows, w.cols
        if not 1 <= m <= NVFP4_MMAX:
            raise ValueError(f"proj_m: M = {m} is outside 1..={NVFP4_MMAX}")
        assert x.is_cuda and x.is_contiguous() and x.numel() == m * k
        if y is None:
            y = torch.empty((m, rows), dtype=torch.float32, device=self.dev)
        name = "gemv_nvfp4_wm" if x.dtype == torch.float32 else "gemv_nvfp4_wm_bf16"
        gx, gy, gz, bx = launch_dims(name, rows, k, m)
        p = self.p
        launch_v(self.k.f(name), gx, gy, gz, bx, [w.w_ptr, x.data_ptr(), w.gs_ptr, y.data_ptr(), p.i32(k), p.i32(rows), p.i32(m)])
        return y

    def gate_up(self, mlp: MlpW, t: int, x: torch.Tensor, h: torch.Tensor | None = None) -> torch.Tensor:
        """h[t][I] = silu(gate x) * up x in one launch (t <= 4)."""
        inter, k = mlp.gate.rows, mlp.gate.cols
        assert (mlp.up.rows, mlp.up.cols) == (inter, k) and x.numel() == t * k and 1 <= t <= NVFP4_MMAX
        if h is None:
            h = torch.empty((t, inter), dtype=torch.float32, device=self.dev)
        p = self.p
        if t == 1:
            name = "gemv_nvfp4_gu" if x.dtype == torch.float32 else "gemv_nvfp4_gu_bf16"
            gx, gy, gz, bx = launch_dims(name, inter, k)
            launch_v(self.k.f(name), gx, gy, gz, bx,
                     [mlp.gate.w_ptr, mlp.up.w_ptr, x.data_ptr(), mlp.gate.gs_ptr, mlp.up.gs_ptr, h.data_ptr(), p.i32(k), p.i32(inter)])
        else:
            name = "gemv_nvfp4_gum" if x.dtype == torch.float32 else "gemv_nvfp4_gum_bf16"
            gx, gy, gz, bx = launch_dims(name, inter, k, t)
            launch_v(self.k.f(name), gx, gy, gz, bx,
                     [mlp.gate.w_ptr, mlp.up.w_ptr, x.data_ptr(), mlp.gate.gs_ptr, mlp.up.gs_ptr, h.data_ptr(), p.i32(k), p.i32(inter), p.i32(t)])
        return h

    def dense_ffn_w(self, mlp: MlpW, x: torch.Tensor, t: int) -> torch.Tensor:
        """down(silu(gate x) * up x) over t <= 4 rows (decode and the MTP verify widths)."""
        h = self.gate_up(mlp, t, x)
        return self.dense_proj(mlp.down, t, h)

    # ------------------------------------------------------------------ head
    def lm_head_row(self, w: Fp4, x: torch.Tensor, fused: bool = True):
        """logits[V] and the greedy token.  fused: one call writes both (the library runs a one-block finishing kernel behind the GEMV);
        else gemv_nvfp4_w + argmax_k over all logits, as the reference."""
        rows, k = w.rows, w.cols
        logits = torch.empty(rows, dtype=torch.float32, device=self.dev)
        idx = torch.zeros(1, dtype=torch.int32, device=self.dev)
        p = self.p
        if fused:
            gx, gy, gz, bx = launch_dims("gemv_nvfp4_w_argmax", rows, k)
            launch_v(self.k.f("gemv_nvfp4_w_argmax"), gx, gy, gz, bx,
                     [w.w_ptr, x.data_ptr(), w.gs_ptr, logits.data_ptr(), p.i32(k), p.i32(rows), idx.data_ptr()])
        else:
            self.dense_proj(w, 1, x, logits.view(1, rows))
            self.argmax(logits, idx)
        return logits, idx

    def argmax(self, logits: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        if out is None:
            out = torch.zeros(1, dtype=torch.int32, device=self.dev)
        launch_v(self.k.f("argmax_k"), 1, 1, 1, 1024, [logits.data_ptr(), out.data_ptr(), self.p.i32(logits.numel())])
        return out

    # ------------------------------------------------------------------ routed experts
    def _check_moe(self, moe: MoeW) -> None:
        """The routed kernels index the table with expert ids of the kernel geometry: a table (or slab tensor) with fewer
        experts would be read past its end.  Refused here, before any launch (the C++ mirror does the same)."""
        e = self.geo.experts
        if moe.gate_up.experts != e or moe.down.experts != e or moe.table.shape[0] != e:
            raise ValueError(f"moe: the geometry has {e} experts, the weights {moe.gate_up.experts} / {moe.down.experts}, the table {moe.table.shape[0]}")

    def router(self, logits: torch.Tensor, moe: MoeW | None = None):
        t, e = logits.shape
        k = self.geo.topk
        if moe is not None:
            self._check_moe(moe)
        assert e == self.geo.experts and logits.dtype == torch.float32 and logits.is_contiguous()
        ids = torch.empty((t, k), dtype=torch.int32, device=self.dev)
        wts = torch.empty((t, k), dtype=torch.float32, device=self.dev)
        gu = torch.zeros((t, k), dtype=torch.int64, device=self.dev)
        dn = torch.zeros((t, k), dtype=torch.int64, device=self.dev)
        table = moe.table.data_ptr() if moe is not None else 0
        launch_v(self.k.f("router_top10"), t, 1, 1, 64,
                 [logits.data_ptr(), 0, ids.data_ptr(), wts.data_ptr(), gu.data_ptr(), dn.data_ptr(), table, 0, 0, 0])
        return ids, wts, gu, dn

    def moe_layer(self, moe: MoeW, x: torch.Tensor, logits: torch.Tensor, y: torch.Tensor | None = None):
        """The routed part of one MoE layer with the launch sequence that is faster for this batch, as measured on MI355X at
        256 experts, top-8: up to 4 tokens the router rides inside the gate|up launch (two launches: 1 token 12.5 us against
        14.1 us for three, 4 tokens 17.8 / 19.8; at 8 tokens every block repeating its token's routing no longer pays); 5 to
        27 tokens per combo in three launches; from 28 grouped by expert (five launches, every expert slab read once per four
        combos: 16 tokens 50 / 57 us per combo / grouped, 24 tokens 69 / 72, 32 tokens 86 / 78, 64 tokens 158 / 101)."""
        if x.shape[0] >= 28:
            return self.moe_run_grouped(moe, x, logits, y)[:3]
        return self.moe_run(moe, x, logits, "route" if x.shape[0] <= 4 else True, y)

    def moe_run_grouped(self, moe: MoeW, x: torch.Tensor, logits: torch.Tensor, y: torch.Tensor | None = None):
        """The routed part of one MoE layer for a batch in which experts repeat: router_top10, moe_group (combos sorted by
        expert, tiles of at most four), then every tile's slab multiplied once by its rows (moe_gate_up_silu_grouped,
        moe_down_grouped) and acc_combo.  The grouping idea of the reference's prefill path (kernels.rs:3322-3384)."""
        t, hdim = x.shape
        inter, topk, experts = self.geo.inter, self.geo.topk, self.geo.experts
        self._check_moe(moe)
        assert hdim == self.geo.hidden and moe.gate_up.rows == 2 * inter and moe.down.rows == hdim
        p = self.p
        ids, wts, _, _ = self.router(logits, moe)
        combos = t * topk
        max_tiles = min(combos, experts) + combos // 4
        if y is None:
            y = torch.zeros((t, hdim), dtype=torch.float32, device=self.dev)
        perm = torch.empty((combos,), dtype=torch.int32, device=self.dev)
        tiles = torch.empty((max_tiles, 4), dtype=torch.int32, device=self.dev)
        n_tiles = torch.zeros((1,), dtype=torch.int32, device=self.dev)
        h2 = torch.empty((combos, inter), dtype=torch.float32, device=self.dev)
        eo = torch.empty((combos, hdim), dtype=torch.float32, device=self.dev)
        table, gs_gu, gs_dn = moe.table.data_ptr(), moe.gate_up.gs.data_ptr(), moe.down.gs.data_ptr()
        launch_v(self.k.f("moe_group"), *launch_dims("moe_group", 1, 64, combos),
                 [ids.data_ptr(), p.i32(combos), perm.data_ptr(), tiles.data_ptr(), n_tiles.data_ptr(), p.i32(max_tiles)])
        launch_v(self.k.f("moe_gate_up_silu_grouped"), *launch_dims("moe_gate_up_silu_grouped", inter, hdim, max_tiles),
                 [tiles.data_ptr(), n_tiles.data_ptr(), perm.data_ptr(), table, x.data_ptr(), gs_gu, h2.data_ptr(),
                  p.i32(hdim), p.i32(topk), p.i32(hdim), p.i32(inter)])
        launch_v(self.k.f("moe_down_grouped"), *launch_dims("moe_down_grouped", hdim, inter, max_tiles),
                 [tiles.data_ptr(), n_tiles.data_ptr(), perm.data_ptr(), table, h2.data_ptr(), gs_dn, eo.data_ptr(), p.i32(inter), p.i32(hdim)])
        launch_v(self.k.f("acc_combo"), (hdim + 255) // 256, t, 1, 256, [eo.data_ptr(), wts.data_ptr(), y.data_ptr()])
        return ids, wts, y, (perm, tiles, n_tiles)

    def moe_run(self, moe: MoeW, x: torch.Tensor, logits: torch.Tensor, fused: bool = True, y: torch.Tensor | None = None):
        """Routed part of one MoE layer: y[t][H] (+)= sum_j w_j * down_e(silu(gate_e x) * up_e x).
        fused=False walks the reference's five launches (router_top10, gemv_fp4_ptrb, silu_mul_combo,
        gemv_fp4_ptrb, acc_combo); fused=True uses router_top10 + moe_gate_up_silu + moe_down_combine; fused="route"
        takes the router into the gate|up launch (moe_route_gate_up_silu + moe_down_combine: two launches)."""
        t, hdim = x.shape
        inter, topk = self.geo.inter, self.geo.topk
        self._check_moe(moe)
        assert hdim == self.geo.hidden and moe.gate_up.rows == 2 * inter and moe.down.rows == hdim
        p = self.p
        combos = t * topk
        if y is None:
            y = torch.zeros((t, hdim), dtype=torch.float32, device=self.dev)
        gs_gu, gs_dn = moe.gate_up.gs.data_ptr(), moe.down.gs.data_ptr()
        h2 = torch.empty((combos, inter), dtype=torch.float32, device=self.dev)
        if fused == "route":
            assert logits.shape == (t, self.geo.experts) and logits.dtype == torch.float32 and logits.is_contiguous()
            ids = torch.empty((t, topk), dtype=torch.int32, device=self.dev)
            wts = torch.empty((t, topk), dtype=torch.float32, device=self.dev)
            dn = torch.zeros((t, topk), dtype=torch.int64, device=self.dev)
            launch_v(self.k.f("moe_route_gate_up_silu"), *launch_dims("moe_route_gate_up_silu", inter, hdim, combos),
                     [logits.data_ptr(), moe.table.data_ptr(), x.data_ptr(), gs_gu, h2.data_ptr(), ids.data_ptr(), wts.data_ptr(), dn.data_ptr(),
                      p.i32(hdim), p.i32(hdim), p.i32(inter)])
            launch_v(self.k.f("moe_down_combine"), *launch_dims("moe_down_combine", hdim, inter, t),
                     [dn.data_ptr(), h2.data_ptr(), gs_dn, wts.data_ptr(), y.data_ptr(), p.i32(inter), p.i32(hdim)])
            return ids, wts, y
        ids, wts, gu, dn = self.router(logits, moe)
        if fused:
            gx, gy, gz, bx = launch_dims("moe_gate_up_silu", inter, hdim, combos)
            launch_v(self.k.f("moe_gate_up_silu"), gx, gy, gz, bx,
                     [gu.data_ptr(), x.data_ptr(), gs_gu, h2.data_ptr(), p.i32(hdim), p.i32(topk), p.i32(hdim), p.i32(inter)])
            launch_v(self.k.f("moe_down_combine"), *launch_dims("moe_down_combine", hdim, inter, t),
                     [dn.data_ptr(), h2.data_ptr(), gs_dn, wts.data_ptr(), y.data_ptr(), p.i32(inter), p.i32(hdim)])
        else:
            h1 = torch.empty((combos, 2 * inter), dtype=torch.float32, device=self.dev)
            eo = torch.empty((combos, hdim), dtype=torch.float32, device=self.dev)
            gx, gy, gz, bx = launch_dims("gemv_fp4_ptrb", 2 * inter, hdim, combos)
            launch_v(self.k.f("gemv_fp4_ptrb"), gx, gy, gz, bx,
                     [gu.data_ptr(), x.data_ptr(), gs_gu, h1.data_ptr(), p.i32(hdim), p.i32(topk), p.i32(hdim), p.i32(2 * inter)])
            n = combos * inter
            launch_v(self.k.f("silu_mul_combo"), (n + 255) // 256, 1, 1, 256, [h1.data_ptr(), h2.data_ptr(), p.i32(n)])
            gx, gy, gz, bx = launch_dims("gemv_fp4_ptrb", hdim, inter, combos)
            launch_v(self.k.f("gemv_fp4_ptrb"), gx, gy, gz, bx,
                     [dn.data_ptr(), h2.data_ptr(), gs_dn, eo.data_ptr(), p.i32(inter), p.i32(1), p.i32(inter), p.i32(hdim)])
            launch_v(self.k.f("acc_combo"), (hdim + 255) // 256, t, 1, 256, [eo.data_ptr(), wts.data_ptr(), y.data_ptr()])
        return ids, wts, y

    # ------------------------------------------------------------------ BF16 keeps (router, q/k, MTP head)
    def bf16_proj(self, w: torch.Tensor, t: int, x: torch.Tensor, y: torch.Tensor | None = None, kernel: str = "gemv_bf16_w") -> torch.Tensor:
        """y[t][rows] = bf16 W [rows][k] times f32 x [t][k]: ``gemv_bf16_w`` (engine/src/kernels.rs:1130-1157), or under the
        names of the reference's block-per-row forms ``gemv_bf16`` (one token) / ``gemv_bf16_b`` (kernels.rs:1061-1098)."""
        assert w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous()
        assert kernel in ("gemv_bf16_w", "gemv_bf16", "gemv_bf16_b", "gemv_bf16_ws")  # _ws: sigmoid at the store (kernels.rs:1430-1458)
        return self._keep_proj(kernel, w, t, x, y)

    def bf16_proj_strided(self, w: torch.Tensor, t: int, x: torch.Tensor, y: torch.Tensor, y_stride: int) -> torch.Tensor:
        """``gemv_bf16_bs`` (kernels.rs:1100-1124): row r of token i lands in y.flatten()[i * y_stride + r] - y may be a view
        that starts inside a wider [t][y_stride] buffer (the shared expert's gate | up pair)."""
        assert w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous()
        rows, k = w.shape
        assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous() and x.numel() == t * k and y.is_cuda and y.dtype == torch.float32
        p = self.p
        launch_v(self.k.f("gemv_bf16_bs"), *launch_dims("gemv_bf16_bs", rows, k, t),
                 [w.data_ptr(), x.data_ptr(), y.data_ptr(), p.i32(k), p.i32(y_stride), p.i32(rows)])
        return y

    def f32_proj(self, w: torch.Tensor, t: int, x: torch.Tensor, y: torch.Tensor | None = None) -> torch.Tensor:
        """y[t][rows] = f32 W [rows][k] times f32 x [t][k]: ``gemv_b``, the router projection (engine/src/gen.rs:4182,
        kernels.rs:97-115); its result is router_top10's logits."""
        assert w.is_cuda and w.dtype == torch.float32 and w.dim() == 2 and w.is_contiguous()
        return self._keep_proj("gemv_b", w, t, x, y)

    def _keep_proj(self, name: str, w: torch.Tensor, t: int, x: torch.Tensor, y: torch.Tensor | None, waves_per_row: int = 0) -> torch.Tensor:
        """waves_per_row: 0 = the library's choice (a block of four waves per row for short tensors), 1 or 4 to force."""
        rows, k = w.shape
        assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous() and x.numel() == t * k
        if y is None:
            y = torch.empty((t, rows), dtype=torch.float32, device=self.dev)
        p = self.p
        launch_v(self.k.f(name), *launch_dims(name, rows, k, t, split=(0, waves_per_row)), [w.data_ptr(), x.data_ptr(), y.data_ptr(), p.i32(k), p.i32(rows)])
        return y

    # ------------------------------------------------------------------ prefill GEMM (M >= 16)
    def gemm(self, w: Fp4, m: int, x: torch.Tensor, y: torch.Tensor | None = None, kernel: str | None = None) -> torch.Tensor:
        """Y[m][rows] = X[m][cols] W^T on the matrix cores (bf16 X, exact bf16 weight tiles, f32 accumulate).
        `kernel` forces one entry point (gemm_nvfp4_bf16_m16 takes m <= 16, the others any m); default: gemm_kernel_for(m, rows)."""
        rows, k = w.rows, w.cols
        assert x.is_cuda and x.is_contiguous() and x.dtype == torch.bfloat16 and x.numel() == m * k
        if y is None:
            y = torch.empty((m, rows), dtype=torch.float32, device=self.dev)
        name = kernel or gemm_kernel_for(m, rows)
        gx, gy, gz, bx = launch_dims(name, rows, k, m)
        p = self.p
        launch_v(self.k.f(name), gx, gy, gz, bx, [w.w_ptr, x.data_ptr(), w.gs_ptr, y.data_ptr(), p.i32(k), p.i32(rows), p.i32(m)])
        return y


def gemm_kernel_for(m: int, rows: int = 17408) -> str:
    """Which GEMM entry point serves m token rows of a [rows, *] tensor: the library's choice (crow_hip_gemm_kernel), which
    weighs how the blocks of each tiling fall on the device's compute units."""
    from . import lib as _l
    return _l.lib().crow_hip_gemm_kernel(rows, m).decode()

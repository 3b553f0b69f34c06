#!/usr/bin/env python3
"""Benchmark of the NVFP4 weight x activation hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-others] [--no-cpu]

One "step" is one pass of benchmark config 1 at batch 1 (M = 1): the fused gate/up + SiLU GEMV
(W_gate, W_up [17408, 5120] NVFP4, X bf16) followed by the down projection (W_down [5120, 17408]
on the f32 H) - the dense FFN of one decode token at the 27B shape.  Weights are N(0, 0.02^2),
seed 0, through the ceil encoder; they are resident in HBM before the timed region and every step
reads a different copy (10 copies, 1.5 GB) so that the 256 MB memory-side cache cannot serve them.
`value` = algorithmic bytes of the step / wall time per step.  The JSON line also carries the
roofline of the dominant kernel (HIP events around back-to-back launches of that kernel alone on
the launch stream), the CPU baseline (the C restatement of the reference's CPU NVFP4 path on this
host's cores: a port, not the Rust binary), and microseconds per call for the other benchmark shapes (configs 0, 2, 3, 4).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_HBM_GBS = 8000.0
REPS = 5  # timing repetitions per figure: the median is reported, the minimum beside it
# HBM bytes per launch of the dominant kernel come from the committed rocprofv3 --pmc summary (FETCH_SIZE / WRITE_SIZE scaled by
# a 256 MiB copy kernel of the same run), keyed by kernel and launch shape: a line
#   TRAFFIC <kernel> grid=<gx>x<slices>x<gz> block=<bx> bytes=<n>
# in this file.  A kernel launched with another shape than the one profiled reports traffic null.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemv_nvfp4_gu_bf16__config1_m1.md")


def traffic_from_profile(kernel: str, dims) -> int | None:
    key = f"TRAFFIC {kernel} grid={dims[0]}x{max(1, dims[1] >> 24)}x{dims[2]} block={dims[3]} bytes="
    try:
        with open(TRAFFIC_PROFILE) as fh:
            for line in fh:
                line = line.strip().strip("`")
                if line.startswith(key):
                    return int(line[len(key):].replace(",", ""))
    except OSError:
        pass
    return None


N, K = 17408, 5120
W_BYTES = N * K // 64 * 36  # 50,135,040: container encoding, 4.5 bits per weight


def alg_bytes_gate_up(m: int, x_bytes: int = 2) -> int:
    return 2 * W_BYTES + m * K * x_bytes + m * N * 4 + 8


def alg_bytes_down(m: int) -> int:
    return W_BYTES + m * N * 4 + m * K * 4 + 4


class Launch:
    """A prepared launch: handle, dims and one ctypes argument array per rotating weight copy."""

    def __init__(self, eng, name, rows, k, z, arg_sets):
        from crow_nest_amd.kernels import launch_dims
        self.f = eng.k.f(name)
        self.dims = launch_dims(name, rows, k, z)
        self.sets = [(C.c_uint64 * len(a))(*[int(v) for v in a]) for a in arg_sets]
        self.raw = arg_sets
        self.n = len(arg_sets[0])

    def go(self, lib, i):
        rc = lib.crow_hip_launch(self.f, *self.dims, self.sets[i % len(self.sets)], self.n, None)
        if rc != 0:
            raise RuntimeError(f"crow_hip_launch failed: {rc}")

    def us(self, iters=200, reps=REPS):
        """(median, minimum) over `reps` repetitions of the mean microseconds per launch of `iters` back-to-back launches."""
        from crow_nest_amd.kernels import time_launches
        time_launches(self.f, *self.dims, self.raw, 20)
        return med_min([time_launches(self.f, *self.dims, self.raw, iters) for _ in range(reps)])


def med_min(ts):
    ts = sorted(ts)
    return ts[len(ts) // 2], ts[0]


# sha256 (first 16 hex digits) of the three container byte strings and of the bf16 activations, recorded from runs in which the
# CPU restatement of the converter's ceiling encoder built the inputs (same generator, same seeds)
CPU_ENCODER_SHA256_16 = {"gate": "fac61cbbd89ba7f6", "up": "c5cddfd1cd12470a", "down": "140d0096e7183bfa", "x_bf16": "efb063872d27b714"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--no-others", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three device copies of 256 MiB (a plain copy kernel of known size) so that a rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE run of this command holds its own scale")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU (every box here has one); --gpus {a.gpus} is not supported. "
              "The path would shard by output rows, with no exchange inside the product.", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from crow_nest_amd import lib as L
    from crow_nest_amd.engine import Engine, gemm_kernel_for
    from crow_nest_amd.kernels import KernelGeo, status
    from crow_nest_amd.weights import load_fp4_quantized, quantize_nvfp4, tiled_bytes
    from oracle import oracle as orc  # the checker of what was timed, and the cpu_baseline leg: never the thing measured
    from refgen import normal_f32

    eng = Engine(KernelGeo(experts=256, topk=8, hidden=2048, inter=512))
    lib = L.lib()
    dev = torch.device("cuda", 0)
    name_buf = C.create_string_buffer(256)
    lib.crow_hip_device_name(name_buf, 256)
    p = eng.p

    # ---------------- synthetic inputs of config 1 (seed 0)
    t0 = time.time()
    host, base = {}, {}
    for i, (nm, rows, cols) in enumerate([("gate", N, K), ("up", N, K), ("down", K, N)]):
        # N(0, 0.02^2) through the library's own encoder (crow_hip_quantize_nvfp4: the converter's ceiling scales, byte for byte)
        blocks, gs_dev = quantize_nvfp4(torch.from_numpy(normal_f32(0, i, rows * cols, 0.02)).to(dev))
        base[nm] = load_fp4_quantized(blocks, gs_dev, rows, cols)
        host[nm] = (blocks.cpu().numpy(), float(gs_dev.cpu().numpy()[0]), rows, cols)  # the container bytes, for the checker and the CPU baseline
        del blocks
    status()
    x32 = normal_f32(0, 10, K)
    xb = torch.from_numpy(x32).to(dev).to(torch.bfloat16)  # round to nearest even
    xb_bits = xb.view(torch.int16).cpu().numpy().view(np.uint16)
    copies = 10
    sets = []
    for c in range(copies):
        sets.append({nm: (base[nm].w.clone() if c else base[nm].w) for nm in base})
    h = torch.empty(N, dtype=torch.float32, device=dev)
    y = torch.empty(K, dtype=torch.float32, device=dev)
    gen_s = time.time() - t0
    import hashlib
    input_sha256 = {nm: hashlib.sha256(host[nm][0].tobytes()).hexdigest()[:16] for nm in host}
    input_sha256["x_bf16"] = hashlib.sha256(xb_bits.tobytes()).hexdigest()[:16]

    gu = Launch(eng, "gemv_nvfp4_gu_bf16", N, K, 1,
                [[s["gate"].data_ptr(), s["up"].data_ptr(), xb.data_ptr(), base["gate"].gs_ptr, base["up"].gs_ptr, h.data_ptr(),
                  p.i32(K), p.i32(N)] for s in sets])
    dn = Launch(eng, "gemv_nvfp4_w", K, N, 1,
                [[s["down"].data_ptr(), h.data_ptr(), base["down"].gs_ptr, y.data_ptr(), p.i32(N), p.i32(K)] for s in sets])

    def step(i):
        gu.go(lib, i)
        dn.go(lib, i)

    if a.copy_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for i in range(a.warmup):
        step(i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for i in range(a.steps):
        step(i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t1
    status()
    ms_per_step = dt * 1e3 / a.steps
    step_bytes = alg_bytes_gate_up(1) + alg_bytes_down(1)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # parity of what was just timed, against the CPU path (the checker, outside the timed region)
    ref_h = orc.silu_mul(orc.gemv(host["gate"][0], N, K, host["gate"][1], orc.bf16_bits_to_f32(xb_bits), threads=8),
                         orc.gemv(host["up"][0], N, K, host["up"][1], orc.bf16_bits_to_f32(xb_bits), threads=8))[0]
    from gpu_common import FLOOR, FLOOR_CHAINED, gamma_rows, rel_err, rel_l2
    gu.go(lib, 0)
    dn.go(lib, 0)
    torch.cuda.synchronize()
    h_dev, y_dev = h.cpu().numpy(), y.cpu().numpy()
    ref_y = orc.gemv(host["down"][0], K, N, host["down"][1], ref_h, threads=8)[0]
    # the down projection alone, on the H the device wrote: one product, so the single-product floor applies to it
    ref_y_dev_h = orc.gemv(host["down"][0], K, N, host["down"][1], h_dev, threads=8)[0]
    r0, nr = 2048, 128  # 128 rows of each product against f64, to be inside the reference's own f32 bound
    y64, ab64 = orc.gemv_f64(host["down"][0], K, N, host["down"][1], h_dev)
    y64, ab64 = y64[0], ab64[0]
    # the whole-tensor rule of tests/test_gpu_full.py: within 1e-3 at the floor, or - for an output that cancelled - the device is
    # the side nearer to f64; every output inside the reference's own bound
    e_abs, e_ref = np.abs(y_dev.astype(np.float64) - ref_y_dev_h), np.abs(ref_y_dev_h.astype(np.float64) - y64)
    rms = float(np.sqrt((ref_y_dev_h.astype(np.float64) ** 2).mean()))
    over = e_abs / np.maximum(np.abs(ref_y_dev_h), FLOOR * rms) > 1e-3
    y_rule = bool(np.all(np.abs(y_dev[over] - y64[over]) <= e_ref[over])) and bool(np.all(np.abs(y_dev - y64) <= orc.gamma(N) * ab64))
    parity = {
        "h_max_rel_err": float(f"{rel_err(h_dev, ref_h):.3g}"), "h_rel_l2": float(f"{rel_l2(h_dev, ref_h):.3g}"),
        "y_on_device_h_max_rel_err": float(f"{rel_err(y_dev, ref_y_dev_h):.3g}"),
        # the same metric against an f64 evaluation of the product, for the device and for the CPU path: outputs that cancel to
        # almost nothing carry either path's f32 summation noise (K = 17408 terms), which is what the figure above compares
        "y_on_device_h_vs_f64_max_rel_err": {"device": float(f"{rel_err(y_dev, y64):.3g}"), "cpu_path": float(f"{rel_err(ref_y_dev_h, y64):.3g}")},
        "y_on_device_h_gamma_ratio_all_rows": float(f"{np.max(np.abs(y_dev - y64) / np.maximum(orc.gamma(N) * ab64, 1e-300)):.3g}"),
        "y_on_device_h_outputs_over_1e-3": int(over.sum()), "y_on_device_h_rule_holds": y_rule,
        "y_chained_max_rel_err": float(f"{rel_err(y_dev, ref_y, FLOOR_CHAINED):.3g}"), "y_chained_rel_l2": float(f"{rel_l2(y_dev, ref_y):.3g}"),
        "denominator_floor": f"max(|ref|, {FLOOR} * rms(ref)) for one product, {FLOOR_CHAINED} * rms for the two products in a row "
                             "(y_chained: H already differs by its own rounding); gamma ratio <= 1 = inside gamma(K/16 + 10) * sum|w x| around f64; "
                             "rule = every output within 1e-3 at the floor or, having cancelled, nearer to f64 on the device than on the CPU path, and all inside the gamma bound",
    }

    # ---------------- the same step as a captured graph (10 steps, one per weight copy, in one graph)
    from crow_nest_amd.kernels import Graph
    gr = Graph()
    with gr.capture():
        for i in range(copies):
            step(i)
    gr.time(3)
    graph_med, graph_min = med_min([gr.time(40) / copies for _ in range(REPS)])
    gr.close()

    # ---------------- roofline of the dominant kernel (gate/up + SiLU), HIP events on the launch stream
    gu_us, gu_us_min = gu.us()
    dn_us, dn_us_min = dn.us()
    gu_bytes = alg_bytes_gate_up(1)
    roof = {"bound": "hbm", "kernel": "gemv_nvfp4_gu_bf16", "achieved": round(gu_bytes / gu_us / 1e3, 1), "peak": PEAK_HBM_GBS,
            "unit": "GB/s", "frac": round(gu_bytes / gu_us / 1e3 / PEAK_HBM_GBS, 4), "traffic": traffic_from_profile("gemv_nvfp4_gu_bf16", gu.dims),
            "traffic_source": "profiles/gemv_nvfp4_gu_bf16__config1_m1.md (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE, scaled by a 256 MiB copy), "
                              "matched on kernel, grid and block; null when the launch shape differs from the profiled one",
            "us_per_launch": round(gu_us, 2), "us_per_launch_min": round(gu_us_min, 2), "timing": f"median (and minimum) of {REPS} x 200 back-to-back launches, HIP events on the launch stream",
            "algorithmic_bytes": gu_bytes, "grid": [gu.dims[0], max(1, gu.dims[1] >> 24), gu.dims[2]], "block": gu.dims[3]}

    # What a PURE READ of the same bytes takes on this chip (nothing else in the kernel): the best of three request patterns - the
    # GEMVs' own 2304-byte groups, and the textbook 16 contiguous bytes per lane with non-temporal and with plain loads - on six
    # grids each (one to seventeen blocks per compute unit, balanced and not), rotating over the same copies.  The gate / up
    # figure reads both tensors' bytes from one buffer of that size.
    from crow_nest_amd.kernels import time_pure_read
    scratch = [torch.empty(2 * tiled_bytes(N, K), dtype=torch.uint8, device=dev) for _ in range(copies)]
    for s_ in scratch:
        s_.random_(0, 64)
    read_only = {}
    for tag, nbytes in (("100MB_gate_up", 2 * tiled_bytes(N, K)), ("50MB_one_tensor", tiled_bytes(N, K))):
        best, by_pattern = None, {}
        ptrs = [s_.data_ptr() for s_ in scratch]
        for pattern, pname in ((0, "groups_as_the_gemv_requests_them"), (1, "16_bytes_per_lane_non_temporal"), (2, "16_bytes_per_lane_plain")):
            for blocks, threads in ((256, 1024), (512, 1024), (1024, 512), (1088, 256), (2176, 256), (4352, 256)):
                time_pure_read(ptrs, nbytes, blocks, threads, 20, pattern)
                us_, us_min_ = med_min([time_pure_read(ptrs, nbytes, blocks, threads, 200, pattern) for _ in range(3)])
                if pname not in by_pattern or us_ < by_pattern[pname]:
                    by_pattern[pname] = round(us_, 2)
                if best is None or us_ < best[0]:
                    best = (us_, us_min_, blocks, threads, pname)
        read_only[tag] = {"us": round(best[0], 2), "us_min": round(best[1], 2), "GB/s": round(nbytes / best[0] / 1e3, 1),
                          "frac_of_peak": round(nbytes / best[0] / 1e3 / PEAK_HBM_GBS, 4), "grid": [best[2], best[3]], "pattern": best[4],
                          "best_us_by_pattern": by_pattern}
    del scratch
    status()
    roof["read_only_same_bytes"] = dict(read_only["100MB_gate_up"], note="a kernel that only reads the two tensors' bytes (best of three request "
                                        "patterns x six grids): the chip's ceiling for this many bytes per launch")
    roof["frac_of_read_only"] = round(read_only["100MB_gate_up"]["us"] / gu_us, 4)

    # config 0 (the reference's own CPU-runnable case): the plain GEMV y = W x on W_gate, f32 x, the same seeded weights
    xk0 = torch.from_numpy(x32).to(dev)
    y0 = torch.empty(N, dtype=torch.float32, device=dev)
    l0 = Launch(eng, "gemv_nvfp4_w", N, K, 1, [[s_["gate"].data_ptr(), xk0.data_ptr(), base["gate"].gs_ptr, y0.data_ptr(), p.i32(K), p.i32(N)] for s_ in sets])
    c0_us, c0_us_min = l0.us()
    c0_bytes = W_BYTES + K * 4 + N * 4 + 4
    torch.cuda.synchronize()
    c0_ref = orc.gemv(host["gate"][0], N, K, host["gate"][1], x32, threads=8)[0]
    c0_y = y0.cpu().numpy()
    config0 = {"workload": "BASELINE config 0: y = W x, W [17408, 5120] NVFP4 (W_gate of config 1), x f32, batch 1",
               "kernel": "gemv_nvfp4_w", "us_per_call": round(c0_us, 2), "us_per_call_min": round(c0_us_min, 2),
               "GB/s": round(c0_bytes / c0_us / 1e3, 1), "pct_of_peak": round(c0_bytes / c0_us / 1e3 / 80, 1), "algorithmic_bytes": c0_bytes,
               "read_only_same_bytes": read_only["50MB_one_tensor"], "frac_of_read_only": round(read_only["50MB_one_tensor"]["us"] / c0_us, 4),
               "parity_max_rel_err": float(f"{rel_err(c0_y, c0_ref):.3g}"), "parity_rel_l2": float(f"{rel_l2(c0_y, c0_ref):.3g}"),
               "gamma_ratio_128_rows": float(f"{gamma_rows(c0_y[r0:r0 + nr], host['gate'][0], r0, nr, K, host['gate'][1], x32):.3g}")}

    out = {
        "metric": "NVFP4 GEMV achieved HBM GB/s (% of peak) and us/call at batch 1, 1 MI355X",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE config 1 at M=1: fused gate/up+SiLU GEMV (W_gate,W_up [17408,5120] NVFP4, X bf16) + down "
                               "projection (W_down [5120,17408] on f32 H), batch 1; 10 rotating weight copies (1.5 GB)",
                   "algorithmic_bytes_per_step": step_bytes, "pct_of_peak": round(100 * value / PEAK_HBM_GBS, 1),
                   "arithmetic": "exact bf16 x bf16 products on the matrix cores (weights decode exactly, f32 activations split "
                                 "into three exact bf16 terms), f32 accumulation and scales",
                   "graph_replay_us_per_step": round(graph_med, 2), "graph_replay_us_per_step_min": round(graph_min, 2),
                   "us_per_call": {"gate_up_silu": round(gu_us, 2), "down": round(dn_us, 2)},
                   "down_frac_of_read_only": round(read_only["50MB_one_tensor"]["us"] / dn_us, 4),
                   "us_per_call_min": {"gate_up_silu": round(gu_us_min, 2), "down": round(dn_us_min, 2)},
                   "parity": parity,
                   "config0": config0,
                   "inputs": {"generator": "splitmix64 + Box-Muller, seed 0, one stream per tensor; W ~ N(0, 0.02^2) through the library's ceiling "
                                           "encoder on the device (crow_hip_quantize_nvfp4), x ~ N(0, 1) rounded to bf16", "sha256_16": input_sha256,
                              # what the CPU restatement of the converter's encoder (and torch's bf16 rounding) gave for the same
                              # streams when it still built these inputs: the device encoder's bytes must be the same bytes
                              "equal_to_the_cpu_encoder_s_bytes": input_sha256 == CPU_ENCODER_SHA256_16,
                              "global_scales": {nm: float(np.float32(host[nm][1])) for nm in host}},
                   "device": name_buf.value.decode(), "input_generation_s": round(gen_s, 1)},
        "roofline": roof,
    }

    # ---------------- the other benchmark shapes: us per call (timing only: random codes, valid scale bytes)
    if not a.no_others:
        others = {}

        def rnd(nbytes):
            return torch.randint(0, 64, (nbytes,), dtype=torch.uint8, device=dev)

        gs1 = torch.tensor([1e-3], dtype=torch.float32, device=dev)
        xf = torch.randn(4, N, device=dev)
        xk = torch.randn(4, K, device=dev)
        xkb = xk.to(torch.bfloat16)
        ybuf = torch.empty(4 * 151936, dtype=torch.float32, device=dev)

        others["note"] = ("timing only: microseconds per call are medians of %d repetitions (us_min beside them); weights of the shapes below "
                          "that are not config 1's own tensors are random bytes (codes and scale bytes 0..63), activations N(0, 1)" % REPS)

        def entry(us, nbytes):
            us, us_min = us
            return {"us": round(us, 2), "us_min": round(us_min, 2), "GB/s": round(nbytes / us / 1e3, 1), "pct_peak": round(nbytes / us / 1e3 / 80, 1)}

        def seq_us(seq, n_sets, iters):
            time_sequence(seq, n_sets, max(n_sets, iters // 10))
            return med_min([time_sequence(seq, n_sets, iters) for _ in range(REPS)])

        # config 0 the reference's way: lanes across the columns, f32 multiply-adds, no matrix instructions, container layout
        # (measurement only: the A/B behind running one activation row on the matrix cores)
        raw = [torch.from_numpy(host["gate"][0]).to(dev) for _ in range(copies)]
        best = None
        for nm in ("gemv_nvfp4_w_valu1", "gemv_nvfp4_w_valu2", "gemv_nvfp4_w_valu4"):
            lv = Launch(eng, nm, N, K, 1, [[r_.data_ptr(), xk0.data_ptr(), base["gate"].gs_ptr, ybuf.data_ptr(), p.i32(K), p.i32(N)] for r_ in raw])
            t_ = lv.us()
            if best is None or t_[0] < best[1][0]:
                best = (nm, t_)
        others["config0_without_matrix_instructions"] = entry(best[1], c0_bytes)
        others["config0_without_matrix_instructions"]["kernel"] = best[0]
        others["config0_without_matrix_instructions"]["vs_matrix_core_kernel"] = round(best[1][0] / c0_us, 2)
        del raw
        # config 1 at verify widths
        for m in (2, 4):
            lg = Launch(eng, "gemv_nvfp4_gum_bf16", N, K, m,
                        [[s["gate"].data_ptr(), s["up"].data_ptr(), xkb.data_ptr(), gs1.data_ptr(), gs1.data_ptr(), ybuf.data_ptr(), p.i32(K), p.i32(N), p.i32(m)] for s in sets])
            ld = Launch(eng, "gemv_nvfp4_wm", K, N, m,
                        [[s["down"].data_ptr(), xf.data_ptr(), gs1.data_ptr(), ybuf.data_ptr(), p.i32(N), p.i32(K), p.i32(m)] for s in sets])
            others[f"config1_gate_up_silu_M{m}"] = entry(lg.us(), alg_bytes_gate_up(m))
            others[f"config1_down_M{m}"] = entry(ld.us(), alg_bytes_down(m))
        # config 3: lm_head + fused argmax
        V = 151936
        vb = tiled_bytes(V, K)
        heads = [rnd(vb) for _ in range(4)]
        idx = torch.zeros(1, dtype=torch.int32, device=dev)
        l3 = Launch(eng, "gemv_nvfp4_w_argmax", V, K, 1, [[hd.data_ptr(), xk.data_ptr(), gs1.data_ptr(), ybuf.data_ptr(), p.i32(K), p.i32(V), idx.data_ptr()] for hd in heads])
        from crow_nest_amd.kernels import time_sequence
        status()
        others["config3_lm_head_151936x5120_argmax"] = entry(l3.us(iters=100), V * K // 64 * 36 + K * 4 + V * 4 + 4)
        others["config3_lm_head_151936x5120_argmax"]["launches"] = "1 call of crow_hip_launch = the GEMV + a one-block finishing kernel"
        lp = Launch(eng, "gemv_nvfp4_w", V, K, 1, [[hd.data_ptr(), xk.data_ptr(), gs1.data_ptr(), ybuf.data_ptr(), p.i32(K), p.i32(V)] for hd in heads])
        others["config3_lm_head_151936x5120_logits_only"] = entry(lp.us(iters=100), V * K // 64 * 36 + K * 4 + V * 4)
        del heads
        # config 4: batched GEMM on the matrix cores
        for m in (16, 128, 512):
            xm = torch.randn(m, K, device=dev).to(torch.bfloat16)
            ym = torch.empty(m, N, dtype=torch.float32, device=dev)
            nm = gemm_kernel_for(m, N)
            l4 = Launch(eng, nm, N, K, m, [[s["gate"].data_ptr(), xm.data_ptr(), gs1.data_ptr(), ym.data_ptr(), p.i32(K), p.i32(N), p.i32(m)] for s in sets])
            us2 = l4.us(iters=50)
            us = us2[0]
            e = entry(us2, W_BYTES + m * K * 2 + m * N * 4)
            e["TFLOP/s"] = round(2.0 * m * N * K / us / 1e6, 1)
            e["pct_mfma_peak_bf16"] = round(2.0 * m * N * K / us / 1e6 / 2500 * 100, 1)
            others[f"config4_gemm_M{m}"] = e
        # BF16 keeps (the tensors the container leaves in bf16): router [256, 2048] and a [10240, 2560] projection, f32 x
        for rows_b, k_b in ((256, 2048), (10240, 2560)):
            n_b = max(2, int(6e8 // (rows_b * k_b * 2)))
            wbs = [torch.randn(rows_b, k_b, device=dev).to(torch.bfloat16) for _ in range(min(n_b, 16))]
            xb_ = torch.randn(k_b, device=dev)
            lb = Launch(eng, "gemv_bf16_w", rows_b, k_b, 1, [[w_.data_ptr(), xb_.data_ptr(), ybuf.data_ptr(), p.i32(k_b), p.i32(rows_b)] for w_ in wbs])
            others[f"bf16_keep_gemv_{rows_b}x{k_b}"] = entry(lb.us(), rows_b * k_b * 2 + k_b * 4 + rows_b * 4)
            del wbs
        # the f32 router projection [256, 2560] (gemv_b: its result is the router's logits)
        wr = [torch.randn(256, 2560, device=dev) for _ in range(16)]
        xr = torch.randn(2560, device=dev)
        lrp = Launch(eng, "gemv_b", 256, 2560, 1, [[w_.data_ptr(), xr.data_ptr(), ybuf.data_ptr(), p.i32(2560), p.i32(256)] for w_ in wr])
        others["f32_router_gemv_256x2560"] = entry(lrp.us(), 256 * 2560 * 4 + 2560 * 4 + 256 * 4)
        del wr
        # config 2: one MoE layer, 256 experts top-8, H 2048, I 512 (router + fused gate|up+SiLU + fused down+combine)
        from crow_nest_amd.engine import MoeW, expert_table
        from crow_nest_amd.weights import ExpertSlabs
        E, H, I = 256, 2048, 512
        sg, sd = tiled_bytes(2 * I, H), tiled_bytes(H, I)
        moes = []
        for _ in range(3):  # 3 x 453 MB of expert slabs
            g_ = ExpertSlabs(rnd(E * sg), gs1, E, 2 * I, H, sg)
            d_ = ExpertSlabs(rnd(E * sd), gs1, E, H, I, sd)
            moes.append(MoeW(g_, d_, expert_table(g_, d_)))
        from crow_nest_amd.kernels import Event
        K8 = 8
        for t in (1, 4):
            xt = torch.randn(t, H, device=dev) * 0.1
            # 24 routing decisions x 3 expert sets: the slabs one step reads (14 MB per token) come round again only after
            # > 256 MB of other slabs, so no step finds its experts in the memory-side cache
            lgs = [torch.randn(t, E, device=dev) for _ in range(24)]
            distinct = sum(len(torch.unique(torch.topk(l_, K8, dim=1).indices)) for l_ in lgs) / len(lgs)
            yt = torch.zeros(t, H, device=dev)
            ids = torch.empty((t, K8), dtype=torch.int32, device=dev)
            wts = torch.empty((t, K8), dtype=torch.float32, device=dev)
            gup = torch.zeros((t, K8), dtype=torch.int64, device=dev)
            dnp = torch.zeros((t, K8), dtype=torch.int64, device=dev)
            h2 = torch.empty((t * K8, I), dtype=torch.float32, device=dev)
            lr = Launch(eng, "router_top10", 1, 64, t, [[l_.data_ptr(), 0, ids.data_ptr(), wts.data_ptr(), gup.data_ptr(), dnp.data_ptr(),
                                                          moes[i_ % 3].table.data_ptr(), 0, 0, 0] for i_, l_ in enumerate(lgs)])
            lgu = Launch(eng, "moe_gate_up_silu", I, H, t * K8, [[gup.data_ptr(), xt.data_ptr(), gs1.data_ptr(), h2.data_ptr(), p.i32(H), p.i32(K8),
                                                                  p.i32(H), p.i32(I)]])
            ldn = Launch(eng, "moe_down_combine", H, I, t, [[dnp.data_ptr(), h2.data_ptr(), gs1.data_ptr(), wts.data_ptr(), yt.data_ptr(), p.i32(I), p.i32(H)]])

            # the layer as Engine.moe_layer runs it at these widths: the router inside the gate|up launch, then down + combine
            lrg = Launch(eng, "moe_route_gate_up_silu", I, H, t * K8,
                         [[l_.data_ptr(), moes[i_ % 3].table.data_ptr(), xt.data_ptr(), gs1.data_ptr(), h2.data_ptr(), ids.data_ptr(), wts.data_ptr(),
                           dnp.data_ptr(), p.i32(H), p.i32(H), p.i32(I)] for i_, l_ in enumerate(lgs)])
            nbytes = int(distinct * (2 * I * H // 64 * 36 + H * I // 64 * 36)) + t * H * 8 + t * E * 4  # every distinct expert once
            for tag, seq in (("", [lrg, ldn]), ("_router_apart", [lr, lgu, ldn])):
                seq2 = [(l_.f, l_.dims, l_.raw) for l_ in seq]
                others[f"config2_moe_layer_T{t}{tag}"] = entry(seq_us(seq2, len(lgs), 240), nbytes)
                others[f"config2_moe_layer_T{t}{tag}"]["launches"] = len(seq)
                others[f"config2_moe_layer_T{t}{tag}"]["distinct_experts_mean"] = round(distinct, 2)
            # the same layer inside a captured graph: 24 consecutive layers (one per routing decision) on one stream per replay
            grm = Graph()
            with grm.capture():
                for i_ in range(len(lgs)):
                    lrg.go(lib, i_)
                    ldn.go(lib, i_)
            grm.time(3)
            g_med, g_min = med_min([grm.time(20) / len(lgs) for _ in range(REPS)])
            grm.close()
            others[f"config2_moe_layer_T{t}"]["graph_replay_24_layers_us_per_layer"] = round(g_med, 2)
            others[f"config2_moe_layer_T{t}"]["graph_replay_24_layers_us_per_layer_min"] = round(g_min, 2)
        # the same layer for a batch in which experts repeat (64 tokens): per combo against grouped by expert
        t = 64
        combos = t * K8
        max_tiles = min(combos, E) + combos // 4
        xt = torch.randn(t, H, device=dev) * 0.1
        yt = torch.zeros(t, H, device=dev)
        lgs = [torch.randn(t, E, device=dev) for _ in range(12)]
        distinct = sum(len(torch.unique(torch.topk(l_, K8, dim=1).indices)) for l_ in lgs) / len(lgs)
        ids = torch.empty((t, K8), dtype=torch.int32, device=dev)
        wts = torch.empty((t, K8), dtype=torch.float32, device=dev)
        gup = torch.zeros((t, K8), dtype=torch.int64, device=dev)
        dnp = torch.zeros((t, K8), dtype=torch.int64, device=dev)
        h2 = torch.empty((combos, I), dtype=torch.float32, device=dev)
        eo = torch.empty((combos, H), dtype=torch.float32, device=dev)
        perm = torch.empty((combos,), dtype=torch.int32, device=dev)
        tiles = torch.empty((max_tiles, 4), dtype=torch.int32, device=dev)
        ntl = torch.zeros((1,), dtype=torch.int32, device=dev)
        lr = Launch(eng, "router_top10", 1, 64, t, [[l_.data_ptr(), 0, ids.data_ptr(), wts.data_ptr(), gup.data_ptr(), dnp.data_ptr(),
                                                      moes[i_ % 3].table.data_ptr(), 0, 0, 0] for i_, l_ in enumerate(lgs)])
        lgu = Launch(eng, "moe_gate_up_silu", I, H, combos, [[gup.data_ptr(), xt.data_ptr(), gs1.data_ptr(), h2.data_ptr(), p.i32(H), p.i32(K8), p.i32(H), p.i32(I)]])
        ldn = Launch(eng, "moe_down_combine", H, I, t, [[dnp.data_ptr(), h2.data_ptr(), gs1.data_ptr(), wts.data_ptr(), yt.data_ptr(), p.i32(I), p.i32(H)]])
        lgr = Launch(eng, "moe_group", 1, 64, combos, [[ids.data_ptr(), p.i32(combos), perm.data_ptr(), tiles.data_ptr(), ntl.data_ptr(), p.i32(max_tiles)]])
        lgg = Launch(eng, "moe_gate_up_silu_grouped", I, H, max_tiles,
                     [[tiles.data_ptr(), ntl.data_ptr(), perm.data_ptr(), moes[i_ % 3].table.data_ptr(), xt.data_ptr(), gs1.data_ptr(), h2.data_ptr(),
                       p.i32(H), p.i32(K8), p.i32(H), p.i32(I)] for i_ in range(len(lgs))])
        ldg = Launch(eng, "moe_down_grouped", H, I, max_tiles,
                     [[tiles.data_ptr(), ntl.data_ptr(), perm.data_ptr(), moes[i_ % 3].table.data_ptr(), h2.data_ptr(), gs1.data_ptr(), eo.data_ptr(),
                       p.i32(I), p.i32(H)] for i_ in range(len(lgs))])
        lac = Launch(eng, "acc_combo", H, 1, t, [[eo.data_ptr(), wts.data_ptr(), yt.data_ptr()]])
        nbytes = int(distinct * (2 * I * H // 64 * 36 + H * I // 64 * 36)) + t * H * 8 + t * E * 4
        for tag, seq in (("per_combo", [lr, lgu, ldn]), ("grouped", [lr, lgr, lgg, ldg, lac])):
            sq = [(l_.f, l_.dims, l_.raw) for l_ in seq]
            others[f"moe_layer_T64_{tag}"] = entry(seq_us(sq, len(lgs), 120), nbytes)
            others[f"moe_layer_T64_{tag}"]["launches"] = len(seq)
        status()
        out["others"] = others

    # ---------------- CPU baseline: the C port of the reference's CPU path on this host (rank 0, N = 1 only)
    if not a.no_cpu:
        threads = max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16), 16))  # the box's CPU share
        units = []
        g = np.random.default_rng(0)
        for u in range(8):  # 8 distinct units of 150 MB: larger than any L3 (the reference's method, cpu_nvfp4.rs:729-777)
            units.append([np.roll(host[nm][0].reshape(-1, 36), 1 + u, axis=0).reshape(-1) if u else host[nm][0] for nm in ("gate", "up", "down")])
        xs = x32.reshape(1, K)
        gsv = [host[nm][1] for nm in ("gate", "up", "down")]
        for u in units:  # warm-up pass
            orc.ffn(u[0], gsv[0], u[1], gsv[1], u[2], gsv[2], K, N, xs, threads=threads, path=1)
        ts = []
        for rep in range(160):
            u = units[rep % 8]
            c0 = time.perf_counter()
            orc.ffn(u[0], gsv[0], u[1], gsv[1], u[2], gsv[2], K, N, xs, threads=threads, path=1)
            ts.append(time.perf_counter() - c0)
        ts.sort()
        med = ts[len(ts) // 2]
        by_threads = {}
        for th in (1, 4, 8):  # the reference reports 1 / 4 / 8 / all threads (cpu_nvfp4.rs:729-777); 64 calls each here
            if th >= threads:
                continue
            tt = []
            for rep in range(64):
                u = units[rep % 8]
                c0 = time.perf_counter()
                orc.ffn(u[0], gsv[0], u[1], gsv[1], u[2], gsv[2], K, N, xs, threads=th, path=1)
                tt.append(time.perf_counter() - c0)
            tt.sort()
            by_threads[str(th)] = round(3 * W_BYTES / tt[len(tt) // 2] / 1e9, 2)
        by_threads[str(threads)] = round(3 * W_BYTES / med / 1e9, 2)
        # every hardware thread the host shows (the reference's own "all threads" leg, cpu_nvfp4.rs:729-777), whatever share of
        # them this process may use: 48 calls
        hw = os.cpu_count() or 1
        best_med, best_threads = med, threads
        if hw > threads:
            th = min(hw, 512)
            for u in units:
                orc.ffn(u[0], gsv[0], u[1], gsv[1], u[2], gsv[2], K, N, xs, threads=th, path=1)
            tt = []
            for rep in range(48):
                u = units[rep % 8]
                c0 = time.perf_counter()
                orc.ffn(u[0], gsv[0], u[1], gsv[1], u[2], gsv[2], K, N, xs, threads=th, path=1)
                tt.append(time.perf_counter() - c0)
            tt.sort()
            by_threads[f"all({th})"] = round(3 * W_BYTES / tt[len(tt) // 2] / 1e9, 2)
            if tt[len(tt) // 2] < best_med:
                best_med, best_threads = tt[len(tt) // 2], th
        cpu_model = "unknown"
        try:
            with open("/proc/cpuinfo") as fh:
                for line in fh:
                    if line.startswith("model name"):
                        cpu_model = line.split(":", 1)[1].strip()
                        break
        except OSError:
            pass
        try:
            usable = len(os.sched_getaffinity(0))
        except (AttributeError, OSError):
            usable = hw
        out["cpu_baseline"] = {"value": round(3 * W_BYTES / best_med / 1e9, 2), "unit": "GB/s", "cores": best_threads, "kind": "port",
                               "ms_per_step": round(best_med * 1e3, 3), "GB/s_by_threads": by_threads,
                               "cpu_model": cpu_model, "hardware_concurrency": hw, "usable_cpus": usable,
                               "sample": "same step (gate/up + SiLU + down, one token, f32 x) on 8 rotating 150 MB weight units, median of 160 calls "
                                         f"at {threads} threads after a warm-up pass, 64 calls for each smaller thread count and 48 with every hardware "
                                         "thread (about 20 core-seconds in all); value = the best of these legs, cores = its thread count; "
                                         "AVX2 path of the C restatement of engine/src/cpu_nvfp4.rs (OpenMP row split)"}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""crow_hip_launch_noalloc (scratch memory in a fixed array inside the library, nothing allocated per call) against
crow_hip_launch (scratch memory from the workspace crow_hip_init allocated): same kernels, same launch dimensions, so the
same bits.  Two calls in a row share the one array, the second with a smaller input; then the fused head, whose keys
live in the same array; then the size limit."""
import numpy as np
import pytest
import torch

from gpu_common import gamma_ratio
from oracle import oracle as orc
from refgen import normal_f32, random_nvfp4

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


def _both(eng, name, dims, vals_of, rows, t=1):
    """One launch through each entry point into fresh outputs filled with a marker; returns the two results."""
    from crow_nest_amd.kernels import launch_noalloc, launch_v
    outs = []
    for launch in (launch_v, launch_noalloc):
        y = torch.full((t, rows), -7.0, dtype=torch.float32, device="cuda")
        launch(eng.k.f(name), *dims, vals_of(y))
        outs.append(y)
    eng.check()
    return [o.cpu().numpy() for o in outs]


def test_split_launches_share_the_static_scratch_two_calls_in_a_row(eng):
    from crow_nest_amd.kernels import launch_dims
    p = eng.p
    # first call: the down projection's shape, 5 column slices per strip (partial sums and arrival counters in scratch);
    # second call, straight after it on the same stream: fewer rows, fewer columns, a different split
    for seed, rows, cols, split in [(11, 1024, 17408, (0, 0)), (12, 304, 5120, (3, 2))]:
        print(f"case rows={rows} cols={cols} split={split}", flush=True)
        w = random_nvfp4(seed, rows, cols)
        gs = 3.1e-4
        x = normal_f32(seed, 1, cols)
        f = _load(w, rows, cols, gs)
        xd = _dev(x)
        dims = launch_dims("gemv_nvfp4_w", rows, cols, 1, split=split)
        assert dims[1] >> 24 > 1  # a split launch: the scratch memory is really used
        a, b = _both(eng, "gemv_nvfp4_w", dims, lambda y: [f.w_ptr, xd.data_ptr(), f.gs_ptr, y.data_ptr(), p.i32(cols), p.i32(rows)], rows)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert gamma_ratio(b[0], w, rows, cols, gs, x) <= 1.0  # and inside the reference's f32 bound around the f64 value


def test_several_activation_rows_through_the_static_scratch(eng):
    from crow_nest_amd.kernels import launch_dims
    p = eng.p
    rows, cols, m = 160, 17408, 3
    w = random_nvfp4(21, rows, cols)
    gs = 2.2e-4
    x = np.stack([normal_f32(22, t, cols) for t in range(m)])
    f = _load(w, rows, cols, gs)
    xd = _dev(x)
    dims = launch_dims("gemv_nvfp4_wm", rows, cols, m)
    assert dims[1] >> 24 > 1
    a, b = _both(eng, "gemv_nvfp4_wm", dims,
                 lambda y: [f.w_ptr, xd.data_ptr(), f.gs_ptr, y.data_ptr(), p.i32(cols), p.i32(rows), p.i32(m)], rows, t=m)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    for t in range(m):
        assert gamma_ratio(b[t], w, rows, cols, gs, x[t]) <= 1.0


def test_fused_head_keeps_its_keys_in_the_static_scratch(eng):
    from crow_nest_amd.kernels import launch_dims, launch_noalloc, launch_v
    p = eng.p
    toks = []
    # twice in a row: the second head (fewer rows) must not see the first one's keys
    for seed, rows, cols in [(31, 4000, 1024), (32, 1000, 512)]:
        w = random_nvfp4(seed, rows, cols)
        gs = 5.0e-4
        x = normal_f32(seed, 1, cols)
        f = _load(w, rows, cols, gs)
        xd = _dev(x)
        dims = launch_dims("gemv_nvfp4_w_argmax", rows, cols)
        res = []
        for launch in (launch_v, launch_noalloc):
            logits = torch.full((rows,), -7.0, dtype=torch.float32, device="cuda")
            tok = torch.full((1,), -1, dtype=torch.int32, device="cuda")
            launch(eng.k.f("gemv_nvfp4_w_argmax"), *dims,
                   [f.w_ptr, xd.data_ptr(), f.gs_ptr, logits.data_ptr(), p.i32(cols), p.i32(rows), tok.data_ptr()])
            res.append((logits.cpu().numpy(), int(tok.item())))
        eng.check()
        (la, ta), (lb, tb) = res
        assert np.array_equal(la.view(np.uint32), lb.view(np.uint32))
        assert ta == tb == orc.argmax_ref(lb)
        toks.append(tb)
    assert toks[1] < 1000


def test_sizes_beyond_the_static_scratch_and_other_kernels_are_refused(eng):
    from crow_nest_amd.kernels import launch_dims, launch_noalloc
    from crow_nest_amd.lib import CrowHipError
    p = eng.p
    rows, cols = 65536 + 16, 17408  # 4097 strips x 5 slices: more strips than counters, more partial sums than 2^20
    dims = launch_dims("gemv_nvfp4_w", rows, cols)
    assert dims[1] >> 24 > 1 and dims[0] > 4096
    dummy = torch.zeros(16, dtype=torch.float32, device="cuda")
    with pytest.raises(CrowHipError) as ei:  # refused on the host: nothing is launched, no pointer is read
        launch_noalloc(eng.k.f("gemv_nvfp4_w"), *dims, [dummy.data_ptr()] * 4 + [p.i32(cols), p.i32(rows)])
    assert ei.value.code == -5
    # partial sums alone: 3500 strips x 5 slices x 64 floats > 2^20, strips within the counters
    rows = 3500 * 16
    dims = launch_dims("gemv_nvfp4_w", rows, cols)
    assert dims[0] == 3500 and dims[0] * (dims[1] >> 24) * 64 > 1 << 20
    with pytest.raises(CrowHipError) as ei:
        launch_noalloc(eng.k.f("gemv_nvfp4_w"), *dims, [dummy.data_ptr()] * 4 + [p.i32(cols), p.i32(rows)])
    assert ei.value.code == -5
    # a fused head of more strips than the static scratch holds keys for (the allocated workspace takes four times as many)
    rows = (16384 + 1) * 16
    dims = launch_dims("gemv_nvfp4_w_argmax", rows, 64)
    with pytest.raises(CrowHipError) as ei:
        launch_noalloc(eng.k.f("gemv_nvfp4_w_argmax"), *dims, [dummy.data_ptr()] * 4 + [p.i32(64), p.i32(rows), dummy.data_ptr()])
    assert ei.value.code == -5
    with pytest.raises(CrowHipError) as ei:  # a kernel that takes no scratch descriptor
        launch_noalloc(eng.k.f("argmax_k"), 1, 1, 1, 1024, [dummy.data_ptr(), dummy.data_ptr(), p.i32(16)])
    assert ei.value.code == -3
    eng.check()

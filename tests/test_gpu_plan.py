"""GPU tests of the prepared cuts ("plan") of the fp16 product: a table, built once per compressed
matrix, of where every wave of the launch starts, so that the kernel has no rows to search for.

Bars: a product with a plan equals the product without one bit for bit (the cuts are the same, so
every row is summed in the same order); the plan itself is a monotone list of (row, row_ptr[row])
from (0, 0) to (rows, stored entries); plans of another size than the launch needs are ignored.
"""
import ctypes

import numpy as np
import pytest
import torch

import macko_spmv
import macko_spmv_amd
from tests import helpers

pytestmark = pytest.mark.gpu

vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64


def _lib():
    lib = ctypes.CDLL(macko_spmv_amd.HIP_LIBRARY_PATH)
    lib.macko_spmv_plan_entries.argtypes = [i32, i32, i64, ctypes.POINTER(i32)]
    lib.macko_spmv_plan_build.argtypes = [vp, i32, i32, i64, vp, i32, vp]
    lib.macko_spmv_f16_planned.argtypes = [vp, vp, vp, vp, i32, vp, vp, i32, i32, i64, vp]
    lib.macko_spmv_f16.argtypes = [vp, vp, vp, vp, vp, i32, i32, i64, vp]
    return lib


def _skewed(rng, rows, cols):
    return helpers.skewed(rng, rows, cols)[0]


CASES = [
    ("uniform", lambda rng: helpers.row_pruned(rng, 4096, 4096, 0.1)),
    ("uniform, long rows", lambda rng: helpers.random_sparse(rng, 3000, 9000, 0.5)),
    ("skewed", lambda rng: _skewed(rng, 14336, 1024)),
    ("skewed, sorted by length", lambda rng: np.ascontiguousarray(
        sorted(_skewed(rng, 6000, 1024), key=lambda row: np.count_nonzero(row)))),
    ("short rows", lambda rng: helpers.random_sparse(rng, 30000, 100, 0.1)),
    ("mostly empty rows", lambda rng: helpers.random_sparse(rng, 50000, 16, 0.02)),
    ("one dense block between empty stretches", None),
    ("tiny", lambda rng: helpers.random_sparse(rng, 5, 64, 0.5)),
]


def _make(label, maker, rng):
    if maker is not None:
        return np.ascontiguousarray(maker(rng), dtype=np.float16)
    dense = np.zeros((9000, 700), dtype=np.float16)
    dense[3000:3400] = (rng.standard_normal((400, 700)) * 0.05).astype(np.float16)
    return dense


@pytest.mark.parametrize("label,maker", CASES, ids=[c[0] for c in CASES])
def test_product_with_plan_equals_product_without(label, maker):
    rng = np.random.default_rng(len(label))
    dense = _make(label, maker, rng)
    rows, cols = dense.shape
    x = rng.standard_normal(cols).astype(np.float16)
    print("plan case", label, dense.shape, flush=True)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    xg = torch.from_numpy(x).cuda()
    lib = _lib()
    P = c[0].numel()
    n = i32(-1)
    assert lib.macko_spmv_plan_entries(rows, cols, P, ctypes.byref(n)) == 0
    assert n.value >= 0 and n.value % 2 == 0
    plan = torch.full((max(n.value, 4),), -7, dtype=torch.int32, device="cuda")
    assert lib.macko_spmv_plan_build(c[2].data_ptr(), rows, cols, P, plan.data_ptr(), n.value, None) == 0
    torch.cuda.synchronize()
    if n.value:
        cuts = plan[:n.value].cpu().numpy().reshape(-1, 2)
        row_ptr = c[2].cpu().numpy()
        assert cuts[0, 0] == 0 and cuts[-1, 0] == rows
        assert np.all(np.diff(cuts[:, 0]) >= 0)
        assert np.array_equal(cuts[:, 1], row_ptr[cuts[:, 0]])
        if rows > len(cuts) - 1:
            # no wave gets more than an even share plus one row's worth of entries and bookkeeping
            per_wave = np.diff(cuts[:, 1]) + 512 * np.diff(cuts[:, 0])
            longest = int(np.diff(row_ptr).max()) + 512
            assert per_wave.max() <= (row_ptr[-1] + 512 * rows) / (len(cuts) - 1) + longest + 1
    # the compiled wrapper attached an equal plan of its own
    attached = getattr(c[2], "_macko_spmv_plan", None)
    assert (attached is None) == (n.value == 0)
    if attached is not None:
        assert torch.equal(attached, plan[:n.value])

    y_plain = torch.full((rows,), 7.0, dtype=torch.float16, device="cuda")
    y_plan = torch.full((rows,), 9.0, dtype=torch.float16, device="cuda")
    assert lib.macko_spmv_f16(c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(), xg.data_ptr(), y_plain.data_ptr(),
                              rows, cols, P, None) == 0
    assert lib.macko_spmv_f16_planned(c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(), plan.data_ptr(), n.value,
                                      xg.data_ptr(), y_plan.data_ptr(), rows, cols, P, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(y_plain.view(torch.int16), y_plan.view(torch.int16))
    helpers.assert_close_fp16(y_plan.cpu().numpy(), helpers.dense_reference(dense, x))
    # through the package: the tuple from compress carries its plan, a bare copy of its tensors does not
    bare = (c[0].clone(), c[1].clone(), c[2].clone(), c[3], c[4])
    assert getattr(bare[2], "_macko_spmv_plan", None) is None
    assert torch.equal(macko_spmv.multiply(c, xg).view(torch.int16), macko_spmv.multiply(bare, xg).view(torch.int16))
    # y = alpha * M x + beta * y
    y0 = rng.standard_normal(rows).astype(np.float16)
    a1, a2 = torch.from_numpy(y0.copy()).cuda(), torch.from_numpy(y0.copy()).cuda()
    macko_spmv.multiply_axpby(c, xg, a1, alpha=0.5, beta=-2.0)
    macko_spmv.multiply_axpby(bare, xg, a2, alpha=0.5, beta=-2.0)
    assert torch.equal(a1.view(torch.int16), a2.view(torch.int16))


def test_shapes_without_a_plan_and_plans_of_another_size():
    lib = _lib()
    n = i32(-1)
    # no stored entries, no rows, fewer rows than waves with long rows, a vector too long for LDS
    for rows, cols, P in [(100, 100, 0), (0, 100, 0), (64, 49152, 64 * 49152 // 2), (4096, 200000, 4096 * 1000)]:
        assert lib.macko_spmv_plan_entries(rows, cols, P, ctypes.byref(n)) == 0
        assert n.value == 0, (rows, cols, P)
    assert lib.macko_spmv_plan_entries(-1, 100, 8, ctypes.byref(n)) != 0
    # a plan of the wrong size is refused when built and ignored when passed to the product
    rng = np.random.default_rng(3)
    dense = helpers.random_sparse(rng, 2000, 512, 0.3)
    x = rng.standard_normal(512).astype(np.float16)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    xg = torch.from_numpy(x).cuda()
    P = c[0].numel()
    assert lib.macko_spmv_plan_entries(2000, 512, P, ctypes.byref(n)) == 0 and n.value > 0
    junk = torch.full((n.value + 64,), 123456, dtype=torch.int32, device="cuda")
    assert lib.macko_spmv_plan_build(c[2].data_ptr(), 2000, 512, P, junk.data_ptr(), n.value + 2, None) != 0
    y1 = torch.empty(2000, dtype=torch.float16, device="cuda")
    y2 = torch.empty(2000, dtype=torch.float16, device="cuda")
    assert lib.macko_spmv_f16_planned(c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(), junk.data_ptr(), n.value + 2,
                                      xg.data_ptr(), y1.data_ptr(), 2000, 512, P, None) == 0
    assert lib.macko_spmv_f16_planned(c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(), None, 0,
                                      xg.data_ptr(), y2.data_ptr(), 2000, 512, P, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(y1, y2)
    helpers.assert_close_fp16(y1.cpu().numpy(), helpers.dense_reference(dense, x))


def test_move_to_device_attaches_a_plan_and_graphs_replay_with_it():
    rng = np.random.default_rng(17)
    dense = _skewed(rng, 8000, 2048)
    x = rng.standard_normal(2048).astype(np.float16)
    on_host = macko_spmv.compress(torch.from_numpy(dense))
    assert getattr(on_host[2], "_macko_spmv_plan", None) is None
    moved = macko_spmv.move_to_device(on_host, "cuda")
    assert getattr(moved[2], "_macko_spmv_plan", None) is not None
    xg = torch.from_numpy(x).cuda()
    eager = macko_spmv.multiply(moved, xg)
    helpers.assert_close_fp16(eager.cpu().numpy(), helpers.dense_reference(dense, x))
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        out = macko_spmv.multiply(moved, xg)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out = macko_spmv.multiply(moved, xg)
        for _ in range(3):
            out.fill_(5.0)
            graph.replay()
            stream.synchronize()
            assert torch.equal(out, eager)
    torch.cuda.current_stream().wait_stream(stream)


def test_a_plan_that_is_not_this_matrix_s_stays_inside_the_arrays():
    # the kernel clamps what it reads from a plan and ends its walk when the rows stop making sense:
    # the product is then wrong, but the call returns, y beyond `rows` is untouched and the next
    # product is right
    rng = np.random.default_rng(23)
    rows, cols = 6000, 1024
    dense = _skewed(rng, rows, cols)
    x = rng.standard_normal(cols).astype(np.float16)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    xg = torch.from_numpy(x).cuda()
    lib = _lib()
    P = c[0].numel()
    good = getattr(c[2], "_macko_spmv_plan")
    n = good.numel()
    cuts = good.view(-1, 2)
    wrong_plans = {
        "reversed": cuts.flip(0).contiguous().view(-1),
        "zeros": torch.zeros_like(good),
        "huge": torch.full_like(good, 1 << 30),
        "negative": torch.full_like(good, -5),
        "rows and entries swapped": cuts.flip(1).contiguous().view(-1),
        "entries of another place": torch.stack([cuts[:, 0], cuts[:, 1].roll(7)], dim=1).contiguous().view(-1),
    }
    for label, plan in wrong_plans.items():
        print("wrong plan:", label, flush=True)
        y = torch.full((rows + 64,), 3.0, dtype=torch.float16, device="cuda")
        assert lib.macko_spmv_f16_planned(c[0].data_ptr(), c[1].data_ptr(), c[2].data_ptr(), plan.data_ptr(), n,
                                          xg.data_ptr(), y.data_ptr(), rows, cols, P, None) == 0
        torch.cuda.synchronize()
        assert bool((y[rows:] == 3.0).all())
    y = macko_spmv.multiply(c, xg)
    helpers.assert_close_fp16(y.cpu().numpy(), helpers.dense_reference(dense, x))


def test_a_row_ptr_that_makes_no_sense_stays_inside_the_arrays():
    # same promise for the kernel's own search (no plan): wrong row_ptr, wrong product, but the call
    # returns and nothing outside y[0 .. rows) is written.  (Shapes whose rows are split between the
    # waves of a workgroup are not part of this test.)
    rng = np.random.default_rng(29)
    rows, cols = 6000, 1024
    dense = helpers.random_sparse(rng, rows, cols, 0.3)
    x = rng.standard_normal(cols).astype(np.float16)
    c = macko_spmv.compress(torch.from_numpy(dense).cuda())
    xg = torch.from_numpy(x).cuda()
    lib = _lib()
    P = c[0].numel()
    good = c[2]
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    wrong = {
        "reversed": good.flip(0).contiguous(),
        "all zero": torch.zeros_like(good),
        "all P": torch.full_like(good, P),
        "random": torch.randint(0, P, good.shape, device="cuda", dtype=torch.int32, generator=g),
        "beyond the arrays": good * 3,
        "negative": -good,
        "sawtooth": (good % 5000).contiguous(),
    }
    for label, row_ptr in wrong.items():
        print("wrong row_ptr:", label, flush=True)
        y = torch.full((rows + 64,), 3.0, dtype=torch.float16, device="cuda")
        assert lib.macko_spmv_f16(c[0].data_ptr(), c[1].data_ptr(), row_ptr.data_ptr(), xg.data_ptr(), y.data_ptr(),
                                  rows, cols, P, None) == 0
        torch.cuda.synchronize()
        assert bool((y[rows:] == 3.0).all())
    y = macko_spmv.multiply((c[0], c[1], c[2].clone(), c[3], c[4]), xg)
    helpers.assert_close_fp16(y.cpu().numpy(), helpers.dense_reference(dense, x))

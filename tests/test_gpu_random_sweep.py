"""Randomized parity sweep on the GPU: every product entry point on a few hundred random shapes and
sparsity patterns (uniform, skewed rows, long gaps that force padding entries, many empty rows),
checked against the dense float64 product of the same fp16 (or int8) data computed by torch on the
GPU, within |err| <= 2e-3 + 1.2e-2 * |want| (the product's stated tolerance plus the rounding of the
fp16 result), and the decompressor against the dense matrix bit for bit.
"""
import pytest
import torch

import macko_spmv as mk

pytestmark = pytest.mark.gpu


def _close(got, want, what, info):
    err = (got.double() - want).abs()
    tol = 2e-3 + 1.2e-2 * want.abs()
    assert bool((err <= tol).all()), (what, info, float((err - tol).max()))


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_and_patterns(seed):
    ops = torch.ops.macko_spmv
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    torch.manual_seed(seed)

    def rnd(lo, hi):
        return int(torch.randint(lo, hi, (1,), generator=gen))

    densities = [0.0, 0.001, 0.01, 0.05, 0.1, 0.3, 0.5, 0.9, 1.0]
    for case in range(100):
        kind = rnd(0, 5)
        if kind == 0:
            rows, cols = rnd(1, 200), rnd(1, 3000)
        elif kind == 1:
            rows, cols = rnd(200, 6000), rnd(8, 600)
        elif kind == 2:
            rows, cols = rnd(1, 40), rnd(3000, 100000)
        elif kind == 3:
            rows, cols = rnd(3000, 30000), rnd(1, 64)
        else:
            rows, cols = rnd(500, 5000), rnd(500, 5000)
        dens = densities[rnd(0, 9)]
        mode = rnd(0, 4)
        info = (seed, case, rows, cols, dens, mode)
        print("sweep case", *info, flush=True)
        W = torch.randn(rows, cols, device="cuda") * 0.05
        mask = torch.rand(rows, cols, device="cuda") < dens
        if mode == 1:    # skewed rows
            mask = torch.rand(rows, cols, device="cuda") < (torch.rand(rows, 1, device="cuda") ** 4 * min(1.0, dens * 4))
        elif mode == 2:  # a long gap in every row
            mask[:, cols // 3: cols // 3 + rnd(0, 700)] = False
        elif mode == 3:  # many empty rows
            mask[torch.rand(rows, device="cuda") < 0.3] = False
        W = torch.where(mask, W, torch.zeros_like(W)).half().contiguous()
        c = mk.compress(W)
        assert torch.equal(mk.decompress(c), W), ("decompress", info)
        x = torch.randn(cols, device="cuda").half()
        Wd = W.double()
        want = Wd @ x.double()
        _close(mk.multiply(c, x), want, "multiply", info)
        y0 = torch.randn(rows, device="cuda").half()
        C = y0.clone()
        mk.multiply_axpby(c, x, C, 0.5, -1.5)
        _close(C, 0.5 * want - 1.5 * y0.double(), "multiply_axpby", info)
        X = torch.randn(rnd(1, 12), cols, device="cuda").half()
        _close(mk.multiply_batched(c, X), X.double() @ Wd.T, "multiply_batched", info)
        if cols % 8 == 0 and cols <= 80000:
            w = (1 + 0.1 * torch.randn(cols, device="cuda")).half()
            xn = ops.decode_rmsnorm(x, w, 1e-5)
            _close(mk.multiply_rmsnorm(c, x, w, 1e-5), Wd @ xn.double(), "multiply_rmsnorm", info)
            gu = torch.randn(2 * cols, device="cuda").half()
            g = ops.decode_silu_mul(gu[:cols], gu[cols:])
            C = y0.clone()
            mk.multiply_silu_mul_axpby(c, gu[:cols], gu[cols:], C, 1.0, 1.0)
            _close(C, Wd @ g.double() + y0.double(), "multiply_silu_mul_axpby", info)
        q = torch.round(W.float() * (127.0 / max(1e-6, float(W.float().abs().max())))).to(torch.int8)
        x8 = (x.float() * 0.01).half()
        _close(mk.multiply_int8(mk.compress_int8(q), x8), q.double() @ x8.double(), "multiply_int8", info)

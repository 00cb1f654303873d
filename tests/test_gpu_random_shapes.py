"""Seeded random problems through the planner's default choice: whatever kernel it picks for a
shape, the result must match the oracle.  Row counts that leave ragged row blocks for every
workgroup shape, K from one tile to long walks (with and without the 64-column tail), every
batch regime, bitwidth, group size and zero-point form."""
import numpy as np
import pytest

from matgptq_amd import _lib
from oracle import matgptq_oracle as o
from tests import _gpu_util as G

pytestmark = pytest.mark.gpu
BITS = (2, 3, 4, 6, 8)


def _cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        b = int(rng.choice(BITS))
        g = int(rng.choice((128, 128, 32, -1)))
        n = 16 * int(rng.integers(1, 41))
        tiles = int(rng.choice((1, 2, 3, 5, 8, 13, 16, 27, 32)))
        k = 128 * tiles + (64 if g != 128 and tiles >= 1 and rng.random() < 0.3 else 0)
        m = int(rng.choice((1, 2, 3, 4, 5, 7, 8, 12, 16, 17, 31, 33, 64, 100, 129, 257)))
        zp = bool(rng.integers(0, 2))
        out.append((b, g, n, k, m, zp))
    return out


@pytest.mark.parametrize("seed", range(6))
def test_random_problems_through_the_default_plan(seed):
    for b, g, n, k, m, zp in _cases(seed, 25):
        lay = G.Layer(n, k, b, g, seed=seed * 1000 + n + k + m, zero_points=zp)
        x = o.make_activations(m, k, seed=seed + m, outlier_frac=0.01)
        plan = _lib.describe_plan(b, g, n, k, m, zp)
        y = lay.run(x)
        what = f"b={b} g={g} N={n} K={k} M={m} zp={zp} [{plan}]"
        G.assert_close_to_oracle(y, x, lay.w, what)
        G.assert_regression_bound(y, x, lay.w, what)


@pytest.mark.parametrize("seed", (20, 21))
def test_random_larger_problems_through_the_default_plan(seed):
    # a few thousand weight rows and batches of hundreds to two thousand rows: the ring tiles, the
    # tiles that split K inside the workgroup and the larger mid-batch shapes; sampled batch rows
    rng = np.random.default_rng(seed)
    for it in range(10):
        b = int(rng.choice(BITS))
        g = int(rng.choice((128, 128, 32, -1)))
        n = 16 * int(rng.choice((64, 100, 160, 256, 288, 384, 512)))
        tiles = int(rng.choice((3, 8, 9, 16, 31, 32)))
        k = 128 * tiles + (64 if g != 128 and rng.random() < 0.2 else 0)
        m = int(rng.choice((130, 250, 384, 500, 512, 640, 777, 1024, 1100, 1536, 2048)))
        zp = bool(rng.integers(0, 2))
        lay = G.Layer(n, k, b, g, seed=1000 * seed + it, zero_points=zp)
        x = o.make_activations(m, k, seed=it + m, outlier_frac=0.01)
        what = f"b={b} g={g} N={n} K={k} M={m} zp={zp} [{_lib.describe_plan(b, g, n, k, m, zp)}]"
        y = lay.run(x)
        rows = np.unique(np.r_[0, m - 1, rng.integers(0, m, 22)])
        G.assert_close_to_oracle(y[rows], x[rows], lay.w, what)
        G.assert_regression_bound(y[rows], x[rows], lay.w, what)


def _bf16_dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(G.DEV)


@pytest.mark.parametrize("seed", (10, 11))
def test_random_problems_bf16_storage(seed):
    import torch
    L = G.lib()
    for b, g, n, k, m, zp in _cases(seed, 20):
        q, s16, z16 = o.make_layer(n, k, g, seed=seed * 1000 + n + k + m, symmetric=not zp)
        s = o.round_to_bf16(s16.astype(np.float32))
        z = z16.astype(np.float32)
        x = o.round_to_bf16(o.make_activations(m, k, seed=seed + m, outlier_frac=0.01).astype(np.float32))
        pk = G.pack_device(q, b, True)

        def reorder(a):
            src = _bf16_dev(a)
            out = torch.empty_like(src)
            _lib.check(L.matgptq_reorder_scales_device(src.data_ptr(), n, k, g, out.data_ptr(), G.stream()))
            return out

        sr = reorder(s)
        zr = reorder(z) if zp else None
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=G.DEV)
        _lib.check(L.matgptq_gemm(b, g, n, k, m, pk.data_ptr(), sr.data_ptr(), zr.data_ptr() if zp else None,
                                  _bf16_dev(x).data_ptr(), y.data_ptr(), G.stream(), 3))
        torch.cuda.synchronize()
        yv = y.float().cpu().numpy()
        ref = o.linear_f64(x, o.dequantize_bf16(q, s, z, b, g))
        what = f"bf16 b={b} g={g} N={n} K={k} M={m} zp={zp} [{_lib.describe_plan(b, g, n, k, m, zp, 3)}]"
        assert np.all(np.isfinite(yv)), what
        assert np.max(np.abs(yv - ref)) <= G.REL_TOL * np.max(np.abs(ref)), what

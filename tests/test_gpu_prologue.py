"""matgptq_gemm_prologue: the batch-1..4 kernel with the operator in front of the linear formed while
the activations are staged (SiLU gate of the fused gate_up output; residual add + RMS norm).  No
counterpart in the reference; checked against the same two steps run separately (the element-wise
operator, then matgptq_gemm) and against the oracle on activations formed on the host."""
import numpy as np
import pytest
import torch

from matgptq_amd import _glue, _lib
from oracle import matgptq_oracle as o
from tests import _gpu_util as G

pytestmark = pytest.mark.gpu

SILU, NORM = 1, 2
BITS = (2, 3, 4, 6, 8)


def prologue(lay, kind, a, b=None, w=None, out=None, eps=1e-5, m=None, flags=1):
    m = a.shape[0] if m is None else m
    y = torch.full((m, lay.n), float("nan"), dtype=torch.float16, device=G.DEV)
    code = G.lib().matgptq_gemm_prologue(
        lay.bits, lay.g, lay.n, lay.k, m, lay.packed.data_ptr(), lay.scales.data_ptr(),
        lay.zeros.data_ptr() if lay.zeros is not None else None, kind, a.data_ptr(),
        b.data_ptr() if b is not None else None, w.data_ptr() if w is not None else None,
        out.data_ptr() if out is not None else None, eps, y.data_ptr(), G.stream(), flags)
    return code, y


def silu_mul_host(gu: np.ndarray) -> np.ndarray:
    f = gu.shape[1] // 2
    g = gu[:, :f].astype(np.float32)
    s = (g / (1.0 + np.exp(-g))).astype(np.float16)
    return (s * gu[:, f:]).astype(np.float16)


def rmsnorm_host(v: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    v32 = v.astype(np.float32)
    rs = 1.0 / np.sqrt(np.mean(v32.astype(np.float64) ** 2, axis=1, keepdims=True) + eps)
    return (v32 * rs.astype(np.float32) * w.astype(np.float32)).astype(np.float16)


@pytest.mark.parametrize("zp", (True, False))
@pytest.mark.parametrize("b", BITS)
def test_silu_gate_in_the_kernel_equals_the_two_steps(b, zp):
    # K = 2560: twenty tiles, five waves; the gate and up halves sit 2560 columns apart in one row
    n, k = 272, 2560
    lay = G.Layer(n, k, b, 128, seed=50 + b, zero_points=zp)
    for m in (1, 2, 3, 4):
        gu = (o.make_activations(m, 2 * k, seed=m) * 1.5).astype(np.float16)
        gud = G.to_dev(gu)
        code, y = prologue(lay, SILU, gud)
        assert code == 0, _lib.load().matgptq_strerror(code)
        act = torch.empty(m, k, dtype=torch.float16, device=G.DEV)
        _glue.silu_mul(gud, act)
        two = G.gemm(b, 128, n, k, act, lay.packed, lay.scales, lay.zeros)
        torch.cuda.synchronize()
        assert torch.equal(y, two), f"b={b} M={m}"  # the same roundings, the same kernel behind them
        G.assert_close_to_oracle(y.cpu().numpy(), silu_mul_host(gu), lay.w, f"silu prologue b={b} M={m}")


def test_silu_gate_on_a_deep_layer_with_two_rounds_and_two_row_blocks():
    # Llama-3-8B's down projection at its real depth (112 tiles: two rounds of sixteen waves), and a
    # layer with many row blocks at M = 4 (two row blocks per workgroup)
    for n, k, m in ((512, 14336, 1), (5280, 512, 4), (5280, 512, 3)):
        lay = G.Layer(n, k, 4, 128, seed=n % 97)
        gu = o.make_activations(m, 2 * k, seed=3)
        code, y = prologue(lay, SILU, G.to_dev(gu))
        assert code == 0
        torch.cuda.synchronize()
        G.assert_close_to_oracle(y.cpu().numpy(), silu_mul_host(gu), lay.w, f"silu prologue {n}x{k} M={m}")
        G.assert_regression_bound(y.cpu().numpy(), silu_mul_host(gu), lay.w, f"silu prologue {n}x{k} M={m}")


@pytest.mark.parametrize("zp", (True, False))
@pytest.mark.parametrize("b", BITS)
def test_add_rmsnorm_in_the_kernel(b, zp):
    n, k, eps = 304, 4096, 1e-5
    lay = G.Layer(n, k, b, 128, seed=70 + b, zero_points=zp)
    rng = np.random.default_rng(b)
    w = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float16)
    wd = G.to_dev(w)
    for m in (1, 2, 3, 4):
        h = (o.make_activations(m, k, seed=10 + m) * 3).astype(np.float16)
        d = o.make_activations(m, k, seed=20 + m)
        hd, dd = G.to_dev(h), G.to_dev(d)
        out = torch.full((m, k), float("nan"), dtype=torch.float16, device=G.DEV)
        code, y = prologue(lay, NORM, hd, dd, wd, out, eps)
        assert code == 0, _lib.load().matgptq_strerror(code)
        torch.cuda.synchronize()
        v = (h + d).astype(np.float16)  # one fp16 rounding, like the residual add it replaces
        assert np.array_equal(out.cpu().numpy(), v), "new residual stream"
        assert torch.equal(hd.cpu(), torch.from_numpy(h)) and torch.equal(dd.cpu(), torch.from_numpy(d))  # inputs untouched
        x = rmsnorm_host(v, w, eps)
        G.assert_close_to_oracle(y.cpu().numpy(), x, lay.w, f"norm prologue b={b} M={m}")
        # the two steps run separately: same values up to the summation order of the mean
        h2, x2 = hd.clone(), torch.empty_like(hd)
        _glue.add_rmsnorm(h2, dd, wd, x2, eps)
        two = G.gemm(b, 128, n, k, x2, lay.packed, lay.scales, lay.zeros)
        torch.cuda.synchronize()
        assert torch.equal(h2, out)
        diff = (y.float() - two.float()).abs().max().item()
        assert diff <= 2e-3 * two.float().abs().max().item(), (b, m, diff)


def test_norm_without_an_added_tensor_and_without_an_output():
    n, k, eps = 6144, 1024, 1e-6
    lay = G.Layer(n, k, 4, 128, seed=5)
    h = o.make_activations(3, k, seed=1)
    w = np.linspace(0.5, 1.5, k).astype(np.float16)
    code, y = prologue(lay, NORM, G.to_dev(h), None, G.to_dev(w), None, eps)  # 384 row blocks at M = 3: two per workgroup
    assert code == 0
    torch.cuda.synchronize()
    G.assert_close_to_oracle(y.cpu().numpy(), rmsnorm_host(h, w, eps), lay.w, "norm only")


def test_limits_and_error_codes():
    lay = G.Layer(64, 256, 4, 128, seed=2)
    a = G.to_dev(o.make_activations(4, 512, seed=1))
    w = G.to_dev(np.ones(256, dtype=np.float16))
    L = G.lib()
    assert prologue(lay, 3, a)[0] == -7                                  # unknown operator
    assert prologue(lay, SILU, a, flags=3)[0] == -7                      # bf16 storage
    assert prologue(lay, SILU, a, flags=1 | (101 << 8))[0] == -7         # forced variants do not apply
    five = G.to_dev(o.make_activations(5, 512, seed=1))
    assert prologue(lay, SILU, five)[0] == -7                            # more than four rows
    assert prologue(lay, NORM, a[:, :256].contiguous(), None, None)[0] == -4   # the norm needs its weight
    h = a[:, :256].contiguous()
    assert prologue(lay, NORM, h, None, w, h)[0] == -11                  # output over the input
    assert "overlaps" in L.matgptq_strerror(-11).decode()
    g32 = G.Layer(64, 256, 4, 32, seed=2)
    assert prologue(g32, SILU, a)[0] == -7                               # group size 32
    deep = G.Layer(16, 128 * 65, 4, 128, seed=3)                         # 65 tiles: not one round
    hd = G.to_dev(o.make_activations(1, 128 * 65, seed=1))
    assert prologue(deep, NORM, hd, None, G.to_dev(np.ones(128 * 65, dtype=np.float16)))[0] == -7
    assert prologue(deep, SILU, G.to_dev(o.make_activations(1, 2 * 128 * 65, seed=1)))[0] == 0
    torch.cuda.synchronize()


def test_prologues_in_a_graph():
    n, k, eps = 512, 2048, 1e-5
    lay = G.Layer(n, k, 3, 128, seed=9)
    h = G.to_dev(o.make_activations(2, k, seed=1))
    d = G.to_dev(o.make_activations(2, k, seed=2))
    w = G.to_dev(np.ones(k, dtype=np.float16))
    out = torch.empty_like(h)
    y = torch.empty(2, n, dtype=torch.float16, device=G.DEV)
    s = torch.cuda.Stream()

    def call():
        _lib.check(G.lib().matgptq_gemm_prologue(3, 128, n, k, 2, lay.packed.data_ptr(), lay.scales.data_ptr(),
                                                lay.zeros.data_ptr(), NORM, h.data_ptr(), d.data_ptr(), w.data_ptr(),
                                                out.data_ptr(), eps, y.data_ptr(), s.cuda_stream, 1))
    with torch.cuda.stream(s):
        call()
        s.synchronize()
        eager = y.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            call()
        for i in range(3):
            y.fill_(float("nan"))
            out.fill_(float("nan"))
            s.synchronize()
            graph.replay()
            s.synchronize()
            assert torch.equal(y, eager), f"replay {i}"
            assert torch.equal(out, h + d)

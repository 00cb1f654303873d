"""n_in_features = 128 t + 64 (the reference packs any multiple of 64,
inference_lib/matgptq_cuda/csrc/utils.cpp:174-184): the tiles are multiplied by the kernel of the
regime, the last 64 columns by a second launch.  Group sizes 32 and -1 (128 cannot divide such K)."""
import numpy as np
import pytest
import torch

import matgptq_amd  # noqa: F401  (registers the torch ops)
from matgptq_amd import _lib
from oracle import matgptq_oracle as o
from tests import _gpu_util as G

pytestmark = pytest.mark.gpu
BITS = (2, 3, 4, 6, 8)


@pytest.mark.parametrize("b", BITS)
def test_device_pack_with_tail_equals_host_pack(b):
    rng = np.random.default_rng(b)
    n, k = 80, 128 * 5 + 64
    q = rng.integers(0, 256, (n, k), dtype=np.uint8)
    L = G.lib()
    for from_master in (True, False):
        codes = q if from_master else o.slice_codes(q, b)
        host = np.zeros(L.matgptq_packed_words(b, n, k), dtype=np.uint32)
        _lib.check(L.matgptq_pack_host(codes.ctypes.data, n, k, b, int(from_master), host.ctypes.data))
        dev = G.pack_device(codes, b, from_master)
        assert np.array_equal(dev.cpu().numpy().view(np.uint32), host)
        back = torch.empty((n, k), dtype=torch.uint8, device=G.DEV)
        _lib.check(L.matgptq_unpack_device(dev.data_ptr(), n, k, b, back.data_ptr(), G.stream()))
        assert np.array_equal(back.cpu().numpy(), o.slice_codes(q, b))


@pytest.mark.parametrize("g", (32, -1))
@pytest.mark.parametrize("zp", (False, True))
@pytest.mark.parametrize("b", BITS)
def test_gemm_with_tail_every_regime(b, zp, g):
    # batch sizes of the gemv, decode, mid-batch and prefill kernels; ragged row blocks
    n, k = 208, 128 * 7 + 64
    lay = G.Layer(n, k, b, g, seed=80 + b, zero_points=zp)
    for m in (1, 3, 4, 7, 16, 40, 300):
        x = o.make_activations(m, k, seed=m + b, outlier_frac=0.01)
        y = lay.run(x)
        G.assert_close_to_oracle(y, x, lay.w, f"b={b} g={g} zp={zp} M={m} {_lib.describe_plan(b, g, n, k, m, zp)}")
        G.assert_regression_bound(y, x, lay.w, f"b={b} g={g} zp={zp} M={m}")


def test_tail_columns_alone_decide_the_output():
    # activations that are zero outside the last 64 columns: the output is the tail product alone,
    # and with 0/1 scales and integer activations it is exact
    rng = np.random.default_rng(3)
    n, k, b, g = 64, 128 * 2 + 64, 4, 32
    codes = rng.integers(0, 1 << b, (n, k), dtype=np.uint8)
    scales = np.round(rng.random((n, k // g))).astype(np.float16)
    pk = G.pack_device(codes, b, from_master=False)
    sd = G.reorder_device(scales, n, k, g)
    w = o.dequantize_kernel_form(codes, scales, b, g)
    for m in (1, 20, 200):
        x = np.zeros((m, k), dtype=np.float16)
        x[:, k - 64:] = np.round(rng.standard_normal((m, 64))).astype(np.float16)
        expect = o.linear_f64(x, w).astype(np.float16)
        y = G.gemm(b, g, n, k, G.to_dev(x), pk, sd, None).cpu().numpy()
        assert np.array_equal(y.view(np.uint16), expect.view(np.uint16)), m
        assert np.any(expect != 0)


@pytest.mark.parametrize("b", (3, 4, 8))
def test_bf16_gemm_with_tail(b):
    n, k, g = 96, 128 * 3 + 64, 32
    q, s16, z16 = o.make_layer(n, k, g, seed=b)
    s = o.round_to_bf16(s16.astype(np.float32))
    z = z16.astype(np.float32)
    pk = G.pack_device(q, b, True)
    w = o.dequantize_bf16(q, s, z, b, g)

    def dev_bf16(a):
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(G.DEV)

    def reorder(a):
        src = dev_bf16(a)
        out = torch.empty_like(src)
        _lib.check(G.lib().matgptq_reorder_scales_device(src.data_ptr(), n, k, g, out.data_ptr(), G.stream()))
        return out

    sr, zr = reorder(s), reorder(z)
    for m in (1, 24, 200):
        x = o.round_to_bf16(o.make_activations(m, k, seed=m).astype(np.float32))
        y = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=G.DEV)
        _lib.check(G.lib().matgptq_gemm(b, g, n, k, m, pk.data_ptr(), sr.data_ptr(), zr.data_ptr(),
                                        dev_bf16(x).data_ptr(), y.data_ptr(), G.stream(), 3))
        torch.cuda.synchronize()
        ref = o.linear_f64(x, w)
        yv = y.float().cpu().numpy()
        assert np.all(np.isfinite(yv))
        assert np.max(np.abs(yv - ref)) <= G.REL_TOL * np.max(np.abs(ref)), (b, m)


@pytest.mark.parametrize("b", BITS)
def test_dense_dequantise_with_tail_is_bit_exact(b):
    n, k, g = 48, 128 * 2 + 64, 32
    q, s, z = o.make_layer(n, k, g, seed=7 * b)
    lay = G.Layer(n, k, b, g, seed=7 * b)
    w = torch.empty((n, k), dtype=torch.float16, device=G.DEV)
    _lib.check(G.lib().matgptq_dequantize_device(b, g, n, k, lay.packed.data_ptr(), lay.scales.data_ptr(),
                                                 lay.zeros.data_ptr(), w.data_ptr(), G.stream()))
    torch.cuda.synchronize()
    assert np.array_equal(w.cpu().numpy().view(np.uint16), lay.w.view(np.uint16))


def test_shapes_the_tail_does_not_cover_are_refused():
    L = G.lib()
    assert L.matgptq_gemm(4, 128, 16, 192, 1, 1, 1, None, 1, 1, None, 1) == -2   # group 128 cannot divide K
    assert L.matgptq_gemm(4, 32, 16, 64, 1, 1, 1, None, 1, 1, None, 1) == -3     # no whole tile
    assert L.matgptq_gemm(4, 32, 16, 224, 1, 1, 1, None, 1, 1, None, 1) == -3    # K % 64 != 0
    assert L.matgptq_master_words(16, 192) == 0
    assert L.matgptq_pack_master_device(1, 16, 192, 1, None) == -3


def test_torch_ops_and_module_with_tail():
    from matgptq_cuda.matgptq_linear import MatGPTQLinear
    n, k, b, g = 64, 128 * 4 + 64, 4, 32
    q, s, z = o.make_layer(n, k, g, seed=21, symmetric=True)
    qs = o.slice_codes(q, b)
    lin = MatGPTQLinear(torch.from_numpy(qs).to(G.DEV), torch.from_numpy(s).to(G.DEV), b, g)
    w = o.dequantize(q, s, z, b, g)
    for m in (1, 33):
        x = o.make_activations(m, k, seed=m)
        y = lin(torch.from_numpy(x).to(G.DEV)).cpu().numpy()
        G.assert_close_to_oracle(y, x, w, f"module M={m}")


def test_gemm_with_tail_in_a_graph():
    # two launches (tiles, then the tail): both capturable; replays, with eager work of the same
    # operator between them, are checked against the eager result
    n, k, b, g = 128, 128 * 6 + 64, 4, 32
    lay = G.Layer(n, k, b, g, seed=5)
    for m in (1, 40):
        x = G.to_dev(o.make_activations(m, k, seed=m))
        eager = G.gemm(b, g, n, k, x, lay.packed, lay.scales, lay.zeros).clone()
        torch.cuda.synchronize()
        stream = torch.cuda.Stream()
        y = torch.empty((m, n), dtype=torch.float16, device=G.DEV)
        with torch.cuda.stream(stream):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                _lib.check(G.lib().matgptq_gemm(b, g, n, k, m, lay.packed.data_ptr(), lay.scales.data_ptr(),
                                                lay.zeros.data_ptr(), x.data_ptr(), y.data_ptr(),
                                                stream.cuda_stream, 1))
            for _ in range(3):
                y.fill_(float("nan"))
                graph.replay()
                stream.synchronize()
                assert torch.equal(y, eager), m
                other = G.gemm(b, g, n, k, x, lay.packed, lay.scales, lay.zeros)
                torch.cuda.synchronize()
                assert torch.equal(other, eager)

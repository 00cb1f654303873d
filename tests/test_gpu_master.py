"""Master-resident bit planes on a real MI355X: the GEMM takes the bitwidth as an argument and
slices in registers.  Integer results bit-exact against the reference's slice; products within
the tolerance of tests/_gpu_util.py; several bitwidths from ONE buffer."""
import numpy as np
import pytest
import torch

import matgptq_cuda  # noqa: F401
import vllm_matgptq
from matgptq_amd import _lib
from oracle import matgptq_oracle as o
from tests import _gpu_util as G

pytestmark = pytest.mark.gpu
BITS = (2, 3, 4, 6, 8)


def planes_device(q: np.ndarray) -> torch.Tensor:
    n, k = q.shape
    out = torch.empty(G.lib().matgptq_master_words(n, k), dtype=torch.int32, device=G.DEV)
    _lib.check(G.lib().matgptq_pack_master_device(G.to_dev(q).data_ptr(), n, k, out.data_ptr(), G.stream()))
    return out


def gemm_master(bits, g, n, k, x, planes, scales, zeros=None, flags=1, workspace="exact"):
    m = x.shape[0]
    L = G.lib()
    y = torch.full((m, n), float("nan"), dtype=torch.float16, device=G.DEV)
    need = L.matgptq_gemm_master_workspace_bytes(bits, g, n, k, m, flags)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=G.DEV) if workspace == "exact" else None
    _lib.check(L.matgptq_gemm_master(bits, g, n, k, m, planes.data_ptr(), scales.data_ptr(),
                                     zeros.data_ptr() if zeros is not None else None, x.data_ptr(), y.data_ptr(),
                                     ws.data_ptr() if ws is not None else None, need if ws is not None else 0,
                                     G.stream(), flags))
    torch.cuda.synchronize()
    return y.cpu().numpy(), need


def test_device_pack_equals_host_pack_and_slices_bit_exactly(golden):
    L = G.lib()
    rng = np.random.default_rng(0)
    n, k = 80, 640
    q = rng.integers(0, 256, (n, k), dtype=np.uint8)
    q[0, :256] = np.arange(256, dtype=np.uint8)
    host = np.zeros(L.matgptq_master_words(n, k), dtype=np.uint32)
    _lib.check(L.matgptq_pack_master_host(q.ctypes.data, n, k, host.ctypes.data))
    dev = planes_device(q)
    assert np.array_equal(dev.cpu().numpy().view(np.uint32), host)
    for i, b in enumerate(BITS):
        back = torch.full((n, k), 0xAA, dtype=torch.uint8, device=G.DEV)
        _lib.check(L.matgptq_unpack_master_device(dev.data_ptr(), n, k, b, back.data_ptr(), G.stream()))
        # the codes the GEMM kernels see: the reference's own slice table, and the oracle
        assert np.array_equal(back.cpu().numpy(), golden["slice_table"][i][q]), b
        assert np.array_equal(back.cpu().numpy(), o.slice_codes(q, b)), b


@pytest.mark.parametrize("g", (128, 32, -1))
@pytest.mark.parametrize("zp", (False, True))
def test_every_bitwidth_from_one_buffer(zp, g):
    # 5 row blocks, 13 K tiles: ragged for two row blocks per workgroup and for the rounds
    n, k = 80, 128 * 13
    q, s, z = o.make_layer(n, k, g, seed=11, symmetric=not zp)
    planes = planes_device(q)
    sc = G.reorder_device(s, n, k, g)
    zr = G.reorder_device(z, n, k, g) if zp else None
    for b in BITS:
        w = o.dequantize(q, s, z, b, g)
        for m in (1, 2, 3, 4):
            x = o.make_activations(m, k, seed=m + b)
            y, need = gemm_master(b, g, n, k, G.to_dev(x), planes, sc, zr)
            assert need == 0  # the kernel reads the planes itself
            G.assert_close_to_oracle(y, x, w, f"master planes b={b} zp={zp} M={m}")
            G.assert_regression_bound(y, x, w, f"master planes b={b} zp={zp} M={m}")
            # the same product on the pre-sliced tensor: same codes, same arithmetic
            y2 = G.gemm(b, g, n, k, G.to_dev(x), G.pack_device(q, b, True), sc, zr).cpu().numpy()
            assert np.max(np.abs(y.astype(np.float64) - y2)) <= 2.0 ** -9 * np.max(np.abs(y2))


def test_exact_in_the_reference_test_regime():
    # 0/1 scales and integer activations: exact arithmetic, the output must equal the closed form
    rng = np.random.default_rng(4)
    n, k = 48, 2048
    q = rng.integers(0, 256, (n, k), dtype=np.uint8)
    scales = np.round(rng.random((n, k // 128))).astype(np.float16)
    planes, sd = planes_device(q), G.reorder_device(scales, n, k, 128)
    for b in BITS:
        w = o.dequantize_kernel_form(o.slice_codes(q, b), scales, b, 128)
        for m in (1, 4):
            x = np.round(rng.standard_normal((m, k))).astype(np.float16)
            y, _ = gemm_master(b, 128, n, k, G.to_dev(x), planes, sd)
            assert np.array_equal(y.view(np.uint16), o.linear_f64(x, w).astype(np.float16).view(np.uint16)), (b, m)


@pytest.mark.parametrize("b,g,m", [(4, 128, 8), (3, 128, 16), (4, 128, 64), (6, 128, 300), (2, 32, 5), (8, -1, 13), (4, 32, 40),
                                   (2, 128, 100), (8, 32, 33), (6, -1, 7), (3, 32, 513), (6, 128, 1000)])
def test_midbatch_kernel_reads_the_planes_itself(b, g, m):
    n, k = 304, 1024
    q, s, z = o.make_layer(n, k, g, seed=b + m)
    planes = planes_device(q)
    sc, zr = G.reorder_device(s, n, k, g), G.reorder_device(z, n, k, g)
    x = o.make_activations(m, k, seed=m)
    # (five to eight batch rows of a layer this small go to the gemv kernel: the mid-batch kernel is
    # forced for them)
    flags = 1 | (82 << 8) if 5 <= m <= 8 and g != 32 else 1
    assert _lib.describe_plan(b, g, n, k, m, True, flags).startswith("midbatch")
    for zeros in (zr, None):
        y, need = gemm_master(b, g, n, k, G.to_dev(x), planes, sc, zeros, flags=flags, workspace=None)
        assert need == 0
        zz = z if zeros is not None else np.full_like(z, 128)
        G.assert_close_to_oracle(y, x, o.dequantize(q, s, zz, b, g), f"planes, mid-batch b={b} g={g} M={m}")
        # bit-identical to the pre-sliced tensor: the same codes reach the same arithmetic
        y2 = G.gemm(b, g, n, k, G.to_dev(x), G.pack_device(q, b, True), sc, zeros, flags=flags).cpu().numpy()
        assert np.array_equal(y, y2)


@pytest.mark.parametrize("b,g,m,n", [(4, 128, 8, 304), (2, 128, 5, 304), (3, -1, 7, 304), (6, 128, 6, 304), (8, -1, 8, 304),
                                     (4, 128, 8, 6144), (8, 128, 7, 6144)])
def test_gemv_kernel_reads_the_planes_at_five_to_eight_rows(b, g, m, n):
    # the instantiation for eight batch rows (one or, from 320 row blocks on, two row blocks per
    # workgroup) on master-resident planes: no workspace, and the result of the pre-sliced tensor
    k = 1024
    q, s, z = o.make_layer(n, k, g, seed=b + m)
    planes = planes_device(q)
    sc, zr = G.reorder_device(s, n, k, g), G.reorder_device(z, n, k, g)
    x = o.make_activations(m, k, seed=m)
    assert _lib.describe_plan(b, g, n, k, m, True).startswith("gemv")
    for zeros in (zr, None):
        y, need = gemm_master(b, g, n, k, G.to_dev(x), planes, sc, zeros, workspace=None)
        assert need == 0
        zz = z if zeros is not None else np.full_like(z, 128)
        G.assert_close_to_oracle(y, x, o.dequantize(q, s, zz, b, g), f"planes, gemv b={b} g={g} M={m}")
        y2 = G.gemm(b, g, n, k, G.to_dev(x), G.pack_device(q, b, True), sc, zeros).cpu().numpy()
        # (the pre-sliced 2-bit tiles pair their octets differently and the 6- and 8-bit ones multiply their two
        # code segments apart: another order of the fp32 sums, so close, not identical)
        assert np.max(np.abs(y.astype(np.float64) - y2)) <= 2.0 ** -9 * np.max(np.abs(y2.astype(np.float64)))


@pytest.mark.parametrize("r,mb", [(1, 1), (2, 1), (4, 1), (1, 2), (2, 2), (4, 2), (1, 4), (2, 4), (4, 4)])
def test_midbatch_kernel_from_planes_every_shape(r, mb):
    # every (row blocks, batch rows) shape of the kernel forced, on codes that hit the rounding
    # carry and the saturation of the slice (all 256 master values occur)
    n, k, m = 208, 128 * 9, 70
    rng = np.random.default_rng(r * 10 + mb)
    q = rng.integers(0, 256, (n, k), dtype=np.uint8)
    q[0, :256] = np.arange(256, dtype=np.uint8)
    _, s, z = o.make_layer(n, k, 128, seed=3)
    planes = planes_device(q)
    sc, zr = G.reorder_device(s, n, k, 128), G.reorder_device(z, n, k, 128)
    x = o.make_activations(m, k, seed=4)
    flags = 1 | ((80 + {1: 0, 2: 1, 4: 2}[r] + 3 * {1: 0, 2: 1, 4: 2}[mb]) << 8)
    for b in BITS:
        y, need = gemm_master(b, 128, n, k, G.to_dev(x), planes, sc, zr, flags=flags, workspace=None)
        assert need == 0
        G.assert_close_to_oracle(y, x, o.dequantize(q, s, z, b, 128), f"planes, mid-batch R{r} mb{mb} b={b}")
        y2 = G.gemm(b, 128, n, k, G.to_dev(x), G.pack_device(q, b, True), sc, zr, flags).cpu().numpy()
        assert np.array_equal(y, y2)


@pytest.mark.parametrize("b,m", [(8, 8), (8, 16), (4, 128), (6, 100), (2, 64)])
def test_many_row_layers_take_the_midbatch_kernel_on_planes(b, m):
    # the plan for the pre-sliced tensor is another kernel here (decode or a prefill tile); on planes the
    # mid-batch kernel saves the slicing pass up to 128 batch rows
    n, k, g = 16384 + 16, 1024, 128
    q, s, z = o.make_layer(n, k, g, seed=b * m)
    planes = planes_device(q)
    sc, zr = G.reorder_device(s, n, k, g), G.reorder_device(z, n, k, g)
    x = o.make_activations(m, k, seed=m)
    y, need = gemm_master(b, g, n, k, G.to_dev(x), planes, sc, zr, workspace=None)
    assert need == 0
    G.assert_close_to_oracle(y, x, o.dequantize(q, s, z, b, g), f"planes, many rows b={b} M={m}")
    G.assert_regression_bound(y, x, o.dequantize(q, s, z, b, g), f"planes, many rows b={b} M={m}")


@pytest.mark.parametrize("b,g,n,k,m", [(8, 128, 304, 1024, 2048), (4, 128, 2048, 1024, 700), (6, 32, 1024, 512, 1500)])
def test_shapes_outside_those_kernels_go_through_the_workspace(b, g, n, k, m):
    q, s, z = o.make_layer(n, k, g, seed=b + m)
    planes = planes_device(q)
    sc, zr = G.reorder_device(s, n, k, g), G.reorder_device(z, n, k, g)
    x = o.make_activations(m, k, seed=m)
    assert _lib.describe_plan(b, g, n, k, m, True).startswith("prefill")
    y, need = gemm_master(b, g, n, k, G.to_dev(x), planes, sc, zr)
    assert need == b * n * k // 8
    rows = np.r_[0:16, m - 16:m]
    G.assert_close_to_oracle(y[rows], x[rows], o.dequantize(q, s, z, b, g), f"workspace path b={b} g={g} M={m}")
    # bit-identical to the pre-sliced tensor: the second launch is the same kernel on the same codes
    y2 = G.gemm(b, g, n, k, G.to_dev(x), G.pack_device(q, b, True), sc, zr).cpu().numpy()
    assert np.array_equal(y, y2)
    with pytest.raises(_lib.MatGPTQError, match="workspace"):
        gemm_master(b, g, n, k, G.to_dev(x), planes, sc, zr, workspace=None)


def test_llama3_8b_layer_full_size_two_bitwidths_from_one_buffer():
    n, k = 6144, 4096
    q, s, z = o.make_layer(n, k, 128, seed=1)
    planes = planes_device(q)
    sc, zr = G.reorder_device(s, n, k, 128), G.reorder_device(z, n, k, 128)
    x = o.make_activations(1, k, seed=2)
    for b in (4, 2):
        y, _ = gemm_master(b, 128, n, k, G.to_dev(x), planes, sc, zr)
        w = o.dequantize(q, s, z, b, 128)
        G.assert_close_to_oracle(y, x, w, f"qkv from planes b={b}")
        G.assert_regression_bound(y, x, w, f"qkv from planes b={b}")


def test_bf16_storage():
    n, k, b = 80, 1024, 3
    q, s16, z16 = o.make_layer(n, k, 128, seed=5)
    s = o.round_to_bf16(s16.astype(np.float32))
    z = z16.astype(np.float32)
    planes = planes_device(q)

    def bf(a):
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(G.DEV)

    sr = torch.ops.matgptq_cuda.reorder_matgptq_scales(bf(s), n, k, 128)
    zr = torch.ops.matgptq_cuda.reorder_matgptq_scales(bf(z), n, k, 128)
    x = o.round_to_bf16(o.make_activations(2, k, seed=3).astype(np.float32))
    y = torch.ops.matgptq_cuda.matmul_matgptq_master(bf(x), planes.view(torch.uint32), sr, zr, n, k, b, 128, 3)
    ref = o.linear_f64(x, o.dequantize_bf16(q, s, z, b, 128))
    assert y.dtype == torch.bfloat16
    assert np.max(np.abs(y.float().cpu().numpy() - ref)) <= G.REL_TOL * np.max(np.abs(ref))


def test_torch_ops_and_plugin_switch_bitwidth_without_moving_anything():
    n, k = 96, 1024
    q, s, z = o.make_layer(n, k, 128, seed=21)
    qd = torch.from_numpy(q).cuda()
    planes = torch.ops.matgptq_cuda.pack_matgptq_master_resident(qd)
    assert planes.dtype == torch.uint32 and planes.numel() == n * k // 4
    assert torch.equal(planes.cpu(), torch.ops.matgptq_cuda.pack_matgptq_master_resident(torch.from_numpy(q)).cpu())
    for b in BITS:
        codes = torch.ops.matgptq_cuda.unpack_matgptq_master_resident(planes, n, k, b)
        assert np.array_equal(codes.cpu().numpy(), o.slice_codes(q, b))
        assert np.array_equal(torch.ops.matgptq_cuda.unpack_matgptq_master_resident(planes.cpu(), n, k, b).numpy(),
                              o.slice_codes(q, b))
    # the plugin with resident planes: the packed slice is never built, switching is a number
    config = vllm_matgptq.MatGPTQConfig(128, 8, 4, "float16", None, resident_master_planes=True)
    layer = torch.nn.Module()
    method = vllm_matgptq.MatGPTQLinearMethod(config)
    method.create_weights(layer, k, [n], k, n, torch.float16)
    layer.cuda()
    layer.qweight.data.copy_(qd)
    layer.scales.data.copy_(torch.from_numpy(s))
    layer.zeros = torch.nn.Parameter(torch.from_numpy(z).cuda(), requires_grad=False)
    method.process_weights_after_loading(layer)
    assert layer.matgptq_weights is None and layer.matgptq_planes.numel() == n * k // 4
    ptr = layer.matgptq_planes.data_ptr()
    for m in (1, 4, 50):  # gemv kernel, and the workspace path through the caching allocator
        x = o.make_activations(m, k, seed=m)
        xd = torch.from_numpy(x).cuda()
        for bits in (4, 2, 8, 3, 6):
            method.set_bitwidth(layer, bits)
            assert layer.matgptq_planes.data_ptr() == ptr
            G.assert_close_to_oracle(method.apply(layer, xd).cpu().numpy(), x, o.dequantize(q, s, z, bits, 128),
                                     f"plugin planes b={bits} M={m}")


def test_master_gemm_in_a_graph():
    # capturable: no allocation besides torch's own, no host reads; replays checked against eager
    n, k = 256, 2048
    q, s, z = o.make_layer(n, k, 128, seed=9)
    planes = torch.ops.matgptq_cuda.pack_matgptq_master_resident(torch.from_numpy(q).cuda())
    sc = torch.ops.matgptq_cuda.reorder_matgptq_scales(torch.from_numpy(s).cuda(), n, k, 128)
    zr = torch.ops.matgptq_cuda.reorder_matgptq_scales(torch.from_numpy(z).cuda(), n, k, 128)
    x = torch.from_numpy(o.make_activations(1, k, seed=1)).cuda()
    eager = {b: torch.ops.matgptq_cuda.matmul_matgptq_master(x, planes, sc, zr, n, k, b, 128, 1).clone() for b in (4, 3)}
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out4 = torch.ops.matgptq_cuda.matmul_matgptq_master(x, planes, sc, zr, n, k, 4, 128, 1)
            out3 = torch.ops.matgptq_cuda.matmul_matgptq_master(x, planes, sc, zr, n, k, 3, 128, 1)
        for _ in range(3):
            out4.fill_(float("nan"))
            out3.fill_(float("nan"))
            graph.replay()
            stream.synchronize()
            assert torch.equal(out4, eager[4]) and torch.equal(out3, eager[3])


@pytest.mark.parametrize("b,m", [(3, 3), (2, 4), (3, 4), (2, 3)])
def test_three_and_four_rows_on_many_row_layers_read_the_planes(b, m):
    # the pre-sliced plan here is the gemv kernel with four row blocks per workgroup, which is not built
    # for planes: on planes the two-row-block shape serves the call, without a workspace
    n, k, g = 16384, 512, 128
    assert "R4" in _lib.describe_plan(b, g, n, k, m, True)
    q, s, z = o.make_layer(n, k, g, seed=b * 7 + m)
    planes = planes_device(q)
    sc, zr = G.reorder_device(s, n, k, g), G.reorder_device(z, n, k, g)
    x = o.make_activations(m, k, seed=m)
    for zeros in (zr, None):
        y, need = gemm_master(b, g, n, k, G.to_dev(x), planes, sc, zeros, workspace=None)
        assert need == 0
        zz = z if zeros is not None else np.full_like(z, 128)
        G.assert_close_to_oracle(y, x, o.dequantize(q, s, zz, b, g), f"planes, gemv R2 b={b} M={m}")

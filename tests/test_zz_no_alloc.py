"""The entry point that allocates nothing (matgptq_gemm_master_static): same result as
matgptq_gemm_master with a caller workspace, on calls that share the library's built-in buffer."""
import numpy as np
import pytest
import torch

from matgptq_amd import _lib
from oracle import matgptq_oracle as o
from tests import _gpu_util as G

pytestmark = pytest.mark.gpu


def _planes(q):
    n, k = q.shape
    out = torch.empty(G.lib().matgptq_master_words(n, k), dtype=torch.int32, device=G.DEV)
    _lib.check(G.lib().matgptq_pack_master_device(G.to_dev(q).data_ptr(), n, k, out.data_ptr(), G.stream()))
    return out


def _case(n, k, m, bits, g, seed):
    q, s, z = o.make_layer(n, k, g, seed=seed)
    return dict(n=n, k=k, m=m, bits=bits, g=g, q=q, s=s, z=z, planes=_planes(q),
                sc=G.reorder_device(s, n, k, g), zr=G.reorder_device(z, n, k, g),
                x=o.make_activations(m, k, seed=seed + 1))


def _with_workspace(c):
    L = G.lib()
    y = torch.full((c["m"], c["n"]), float("nan"), dtype=torch.float16, device=G.DEV)
    need = L.matgptq_gemm_master_workspace_bytes(c["bits"], c["g"], c["n"], c["k"], c["m"], 1)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device=G.DEV)
    _lib.check(L.matgptq_gemm_master(c["bits"], c["g"], c["n"], c["k"], c["m"], c["planes"].data_ptr(),
                                     c["sc"].data_ptr(), c["zr"].data_ptr(), G.to_dev(c["x"]).data_ptr(),
                                     y.data_ptr(), ws.data_ptr(), need, G.stream(), 1))
    torch.cuda.synchronize()
    return y.cpu().numpy(), need


def _static(c, y=None, xd=None):
    L = G.lib()
    y = torch.full((c["m"], c["n"]), float("nan"), dtype=torch.float16, device=G.DEV) if y is None else y
    xd = G.to_dev(c["x"]) if xd is None else xd
    _lib.check(L.matgptq_gemm_master_static(c["bits"], c["g"], c["n"], c["k"], c["m"], c["planes"].data_ptr(),
                                            c["sc"].data_ptr(), c["zr"].data_ptr(), xd.data_ptr(), y.data_ptr(),
                                            G.stream(), 1))
    torch.cuda.synchronize()
    return y.cpu().numpy()


def test_static_workspace_entry_point_two_calls_in_a_row():
    # first a large input, then a smaller one: the second call finds the first call's sliced
    # tensor in the shared buffer and must not be disturbed by it
    # (batches of more than a thousand rows: the kernels for smaller ones read the planes themselves)
    big = _case(1024, 4096, 1100, 6, 128, seed=1)   # 3 MiB of sliced codes
    small = _case(768, 1024, 1500, 3, 32, seed=2)   # 288 KiB, group 32
    for c in (big, small, big, small):
        want, need = _with_workspace(c)
        assert need == c["bits"] * c["n"] * c["k"] // 8 > 0
        got = _static(c)
        assert np.array_equal(got, want)  # same kernels on the same sliced codes: same bits
        rows = np.r_[0:24, c["m"] - 24:c["m"]]
        G.assert_close_to_oracle(got[rows], c["x"][rows], o.dequantize(c["q"], c["s"], c["z"], c["bits"], c["g"]),
                                 f"static workspace N={c['n']} b={c['bits']}")


def test_static_entry_point_without_scratch_use_and_limits():
    # batch 1..4 reads the planes in the kernel: no scratch involved
    c = _case(256, 2048, 1, 4, 128, seed=3)
    want, need = _with_workspace(c)
    assert need == 0
    assert np.array_equal(_static(c), want)
    # a sliced tensor beyond the built-in buffer is refused with its own error, nothing is launched
    L = G.lib()
    code = L.matgptq_gemm_master_static(8, 128, 28672, 4096, 2048, 1, 1, None, 1, 1, None, 1)
    assert code == -10 and "built-in workspace" in L.matgptq_strerror(code).decode()


def test_static_entry_point_under_graph_capture():
    # what it is for: a captured region may not allocate
    c = _case(512, 2048, 1200, 4, 128, seed=5)
    want, _ = _with_workspace(c)
    assert np.array_equal(_static(c), want)  # first call on the device: outside the capture
    xd = G.to_dev(c["x"])
    y = torch.full((c["m"], c["n"]), float("nan"), dtype=torch.float16, device=G.DEV)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            _lib.check(G.lib().matgptq_gemm_master_static(
                c["bits"], c["g"], c["n"], c["k"], c["m"], c["planes"].data_ptr(), c["sc"].data_ptr(),
                c["zr"].data_ptr(), xd.data_ptr(), y.data_ptr(), stream.cuda_stream, 1))
        for _ in range(3):
            y.fill_(float("nan"))
            graph.replay()
            stream.synchronize()
            assert np.array_equal(y.cpu().numpy(), want)

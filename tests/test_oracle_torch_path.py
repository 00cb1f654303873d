"""The torch restatement used as CPU baseline against the NumPy oracle and the golden vectors."""
import numpy as np
import pytest
import torch

from oracle import matgptq_oracle as o, torch_path as tp

BITS = (2, 3, 4, 6, 8)


@pytest.mark.parametrize("b", BITS)
def test_torch_path_matches_golden(b, golden):
    q, s, z = (torch.from_numpy(golden[k]) for k in ("q", "scale", "zero"))
    w = tp.get_weight(q, s, z, 8, b)
    assert np.array_equal(w.numpy().view(np.uint16), golden[f"w_b{b}"].view(np.uint16))
    y = tp.forward(torch.from_numpy(golden["x"]), q, s, z, 8, b)
    assert np.array_equal(y.numpy().view(np.uint16), golden[f"y_b{b}"].view(np.uint16))
    x = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    assert np.array_equal(tp.matryoshka_slice(x, 8, b).numpy(), golden["slice_table"][BITS.index(b)])


@pytest.mark.parametrize("g", (128, 32))
def test_torch_path_matches_numpy_oracle(g):
    q, s, z = o.make_layer(64, 512, g, seed=11)
    x = o.make_activations(2, 512, seed=11)
    for b in BITS:
        w = tp.get_weight(torch.from_numpy(q), torch.from_numpy(s), torch.from_numpy(z), 8, b)
        assert np.array_equal(w.numpy().view(np.uint16), o.dequantize(q, s, z, b, g).view(np.uint16))
        y = tp.forward(torch.from_numpy(x), torch.from_numpy(q), torch.from_numpy(s), torch.from_numpy(z), 8, b)
        ref = o.linear_f64(x, o.dequantize(q, s, z, b, g))
        assert np.max(np.abs(y.numpy() - ref)) <= 2e-3 * np.max(np.abs(ref))

"""bitnet_hip_bitlinear_forward_noalloc: the forward with its scratch in the library's static per-GPU array.
Checked through the C ABI against bitnet_hip_bitlinear_forward, bit for bit, on consecutive calls that share
the array (the later ones smaller than the earlier ones), and at the limits of the array."""
import numpy as np
import pytest
import torch

import bitnet_hip as bh
from helpers import synth_activations, synth_weights

pytestmark = pytest.mark.gpu


def _layer(rng, n, k):
    layer = bh.BitLinear(bh.BitLinearConfig(in_features=k, out_features=n), "noalloc")
    layer.update_weights(torch.from_numpy(synth_weights(rng, n, k)).cuda())
    return layer


@pytest.mark.parametrize("n,k,rows", [(640, 2560, (64, 7)), (2560, 6912, (151, 33, 8)), (6912, 2560, (256, 96, 2)),
                                      (48, 300, (40, 9))])
def test_forward_noalloc_matches_forward_on_consecutive_calls(n, k, rows):
    bh.init(0)
    rng = np.random.default_rng(n + k)
    layer = _layer(rng, n, k)
    gamma = torch.from_numpy((1 + 0.1 * rng.standard_normal(k)).astype(np.float32)).cuda()
    for use_gamma in (False, True):
        for m in rows:  # the second and third calls are smaller: the array still holds the previous call's rows
            x = torch.from_numpy(synth_activations(rng, m, k, outliers=True)).cuda()
            res = torch.from_numpy(synth_activations(rng, m, n)).cuda()
            g = gamma if use_gamma else None
            want = layer.forward(x, gamma=g, residual=res)
            out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
            got = layer.forward_noalloc(x, out, gamma=g, residual=res)
            torch.cuda.synchronize()
            assert got.data_ptr() == out.data_ptr()
            assert torch.equal(got.view(torch.int32), want.view(torch.int32)), f"m={m} gamma={use_gamma}"


def test_forward_noalloc_allocates_nothing_and_rejects_what_does_not_fit():
    bh.init(0)
    rng = np.random.default_rng(3)
    layer = _layer(rng, 64, 1024)
    x = torch.from_numpy(synth_activations(rng, 16, 1024)).cuda()
    out = torch.empty((16, 64), dtype=torch.float32, device="cuda")
    layer.forward_noalloc(x, out)  # first use on this device done
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(20):
        layer.forward_noalloc(x, out)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    # rank 3 input is flattened like forward's
    x3 = x.view(2, 8, 1024)
    out3 = torch.empty((2, 8, 64), dtype=torch.float32, device="cuda")
    layer.forward_noalloc(x3, out3)
    assert torch.equal(out3.view(16, 64), layer.forward(x))
    # the largest call that fits: 1024 rows x 1024 features
    big = torch.from_numpy(synth_activations(rng, 1024, 1024)).cuda()
    out_big = torch.empty((1024, 64), dtype=torch.float32, device="cuda")
    layer.forward_noalloc(big, out_big)
    assert torch.equal(out_big, layer.forward(big))
    # one row more does not
    too_big = torch.zeros((1025, 1024), dtype=torch.float32, device="cuda")
    with pytest.raises(bh.BitLinearError) as ei:
        layer.forward_noalloc(too_big, torch.empty((1025, 64), dtype=torch.float32, device="cuda"))
    assert ei.value.kind == "MemoryError" and "static scratch" in str(ei.value)
    narrow = _layer(rng, 16, 4)
    many = torch.zeros((4097, 4), dtype=torch.float32, device="cuda")
    with pytest.raises(bh.BitLinearError) as ei:
        narrow.forward_noalloc(many, torch.empty((4097, 16), dtype=torch.float32, device="cuda"))
    assert ei.value.kind == "MemoryError"
    # shape errors as in forward
    with pytest.raises(bh.BitLinearError) as ei:
        layer.forward_noalloc(torch.zeros((2, 5), device="cuda"), torch.empty((2, 64), device="cuda"))
    assert ei.value.kind == "ShapeMismatch"
    # and a small call after the large one still matches
    layer.forward_noalloc(x, out)
    assert torch.equal(out, layer.forward(x))

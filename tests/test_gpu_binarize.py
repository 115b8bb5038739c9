"""GPU parity of the input binarisation kernels against the oracle's restatement of
src/convlogic/data.py:46-71 (bit-exact: the kernels only compare)."""
import numpy as np
import pytest
import torch

import convlogic_amd as C
from convlogic_amd.convlogic import binarize
from convlogic_amd.hip import convlogic_hip
from oracle import convlogic_oracle as O
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,c0,h,w,levels", [(1, 1, 1, 1, 1), (70, 3, 5, 7, 3), (64, 1, 28, 28, 1), (200, 3, 32, 32, 3), (33, 2, 4, 4, 9)])
def test_threshold_float_and_packed_match_oracle(n, c0, h, w, levels):
    torch.manual_seed(n + levels)
    x = torch.rand(n, c0, h, w)
    thr = O.thresholds_uniform(levels)
    x[0, 0, 0, 0] = thr[0]                                         # equality is not "greater"
    want = O.apply_thresholds(x, thr)
    got = binarize.apply_thresholds(x.to(DEV), thr)
    assert got.dtype == torch.float32 and torch.equal(got.cpu(), want)
    assert torch.equal(binarize.apply_thresholds(x, thr), want)    # host tensors: torch expression
    assert torch.equal(binarize.apply_thresholds(x[0].to(DEV), thr).cpu(), O.apply_thresholds(x[0], thr))
    p = binarize.pack_thresholds(x.to(DEV), thr)
    words, pad = O.pack_image(want.numpy() > 0.5)
    assert p.image and p.bit_count == 64 and p.pad_len == pad
    assert np.array_equal(p.t.cpu().numpy(), words)
    ref = C.PackBitsTensor(want.bool().to(DEV), 64)
    assert torch.equal(ref.t, p.t)


def test_thresholds_and_network_input():
    torch.manual_seed(1)
    assert torch.equal(binarize.uniform_thresholds(3), O.thresholds_uniform(3))
    data = torch.rand(50, 3, 8, 8)
    assert torch.equal(binarize.distributive_thresholds(data, 4), O.thresholds_distributive(data, 4))
    assert torch.equal(binarize.compute_thresholds(data, "Uniform", 2), O.thresholds_uniform(2))
    with pytest.raises(ValueError):
        binarize.compute_thresholds(data, "median", 2)
    # BASELINE config 4/5 input: N(0.5, 0.25) clipped, thresholds 0.25/0.5/0.75 -> 9 channels; packed input == float input
    v = (torch.randn(100, 3, 32, 32) * 0.25 + 0.5).clamp(0, 1).to(DEV)
    thr = binarize.uniform_thresholds(3)
    model = C.ConvLogicCifarModel(k_param=4, input_channels=9, tau=6.5).to(DEV).eval()
    with torch.no_grad():
        y = model(binarize.apply_thresholds(v, thr))
        counts = model(binarize.pack_thresholds(v, thr))
    assert torch.equal(counts.float(), torch.round(y * 6.5))


def test_threshold_errors():
    x = torch.rand(4, 3, 8, 8, device=DEV)
    thr = torch.tensor([0.5], device=DEV)
    with pytest.raises(RuntimeError):
        convlogic_hip.threshold_images(x.double(), thr)
    with pytest.raises(RuntimeError):
        convlogic_hip.threshold_pack_images(x[0], thr)
    with pytest.raises(NotImplementedError):
        binarize.pack_thresholds(x.cpu(), thr.cpu())

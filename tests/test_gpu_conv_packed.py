"""GPU parity of the packed-bit conv-logic block (64 samples per word, group-major images): bit-exact
against the numpy oracle and against the float eval path on the same binary inputs.  The reference has
no packed conv path; the oracle is pinned in tests/test_oracle.py by the float eval-mode block."""
import numpy as np
import pytest
import torch

import convlogic_amd as C
from convlogic_amd.hip import convlogic_hip
from oracle import convlogic_oracle as O
from tests.gpu_util import DEV, set_knobs

pytestmark = pytest.mark.gpu
GEOMS = [(1, 1, 3), (2, 2, 4), (1, 0, 3), (2, 1, 3), (1, 2, 5)]


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def _layer(cin, cout, stride, pad, kernel, seed, selection=None):
    torch.manual_seed(seed)
    layer = C.ConvLogicLayer(cin, cout, stride=stride, padding=pad, kernel=kernel, complete=True, implementation="cuda",
                             selection=selection).to(DEV)
    with torch.no_grad():
        layer.weights.copy_(torch.randn_like(layer.weights))
    return layer.eval()


def _fit_even(h, w, stride, pad, kernel):
    ho, wo = O.conv_out_size(h, w, _pair(stride), _pair(pad), _pair(kernel))
    return h + (ho % 2) * _pair(stride)[0], w + (wo % 2) * _pair(stride)[1]


@pytest.mark.parametrize("stride,pad,kernel", GEOMS)
@pytest.mark.parametrize("n", [1, 64, 130])
@pytest.mark.parametrize("subset", [None, "1", "direct"])
def test_packed_block_small_vs_oracle(stride, pad, kernel, n, subset, monkeypatch):
    if subset == "1":
        set_knobs(monkeypatch, CLG_FWD_SUBSET="1")          # two LDS planes per kernel instead of all channels
        set_knobs(monkeypatch, CLG_FWD_DIRECT="0")
    if subset == "direct":
        set_knobs(monkeypatch, CLG_FWD_DIRECT="1")          # taps from a padded global copy, no LDS
    cin, cout = 3, 6
    h, w = _fit_even(8 + pad, 10 + pad, stride, pad, kernel)
    layer = _layer(cin, cout, stride, pad, kernel, seed=n + stride)
    bits = torch.randint(0, 2, (n, cin, h, w), device=DEV).bool()
    p = C.PackBitsTensor(bits, 64)
    want_words, want_pad = O.pack_image(bits.cpu().numpy())
    assert p.image and p.pad_len == want_pad and np.array_equal(p.t.cpu().numpy(), want_words)
    out = layer(p)
    assert out is p and p.image
    gates = layer.weights.argmax(-1).to(torch.uint8).cpu().numpy()
    want = O.conv_block_eval_packed(want_words, gates, layer.selection.cpu().numpy(), _pair(stride), _pair(pad), _pair(kernel))
    got = p.t.cpu().numpy()
    assert got.shape == want.shape and got.dtype == np.int64
    # bits of the padding samples are whatever the gates make of zeros; compare the real samples
    assert np.array_equal(O.unpack_image(got, want_pad), O.unpack_image(want, want_pad))
    assert np.array_equal(got, want)                        # and the padding bits, too: same arithmetic


@pytest.mark.parametrize("shape", [(200, 9, 32, 32, 32), (200, 32, 128, 16, 16), (130, 128, 512, 8, 8), (130, 512, 1024, 4, 4),
                                   (70, 1, 32, 28, 28), (64, 200, 40, 16, 16), (300, 24, 48, 4, 4), (65, 6, 12, 2, 2)])
def test_packed_block_equals_float_eval_path(shape):
    # blocks of BASELINE config 5 / 3 and shapes beyond the LDS plans: the float kernels (checked against the
    # oracle elsewhere) give exactly 0/1 on binary inputs in eval mode; the packed block must give the same bits
    n, cin, cout, h, w = shape
    layer = _layer(cin, cout, 1, 1, 3, seed=cin)
    bits = torch.randint(0, 2, (n, cin, h, w), device=DEV).bool()
    with torch.no_grad():
        y = layer(bits.float())
    assert torch.all((y == 0) | (y == 1))
    p = layer(C.PackBitsTensor(bits, 64))
    got = O.unpack_image(p.t.cpu().numpy(), p.pad_len)
    assert np.array_equal(got, y.cpu().numpy() > 0.5)


@pytest.mark.parametrize("subset", ["0", "1"])
def test_selection_with_more_than_two_channels_per_kernel(subset, monkeypatch):
    set_knobs(monkeypatch, CLG_FWD_DIRECT="0")
    # a caller-made selection may name up to 8 channels per kernel; the two-planes-per-kernel staging then
    # reads those kernels' taps from global memory (float and packed)
    set_knobs(monkeypatch, CLG_FWD_SUBSET=subset)
    torch.manual_seed(2)
    cin, cout, h, w = 12, 10, 8, 8
    ch = torch.randint(0, cin, (cout, 8))
    ch[::2] = ch[::2, :1]                                   # every other kernel keeps a single channel
    sel = ((ch << 16) | (torch.randint(0, 3, (cout, 8)) << 8) | torch.randint(0, 3, (cout, 8))).to(torch.int32)
    layer = _layer(cin, cout, 1, 1, 3, seed=5, selection=sel.to(DEV))
    bits = torch.randint(0, 2, (100, cin, h, w), device=DEV).bool()
    gates = layer.weights.argmax(-1).to(torch.uint8).cpu().numpy()
    words, pad = O.pack_image(bits.cpu().numpy())
    want = O.conv_block_eval_packed(words, gates, sel.numpy(), (1, 1), (1, 1), (3, 3))
    p = layer(C.PackBitsTensor(bits, 64))
    assert np.array_equal(p.t.cpu().numpy(), want)
    with torch.no_grad():
        y = layer(bits.float())
    assert np.array_equal(y.cpu().numpy() > 0.5, O.unpack_image(want, pad))
    # training-mode float forward on real inputs through the same staging
    layer.train()
    x = torch.rand(5, cin, h, w, device=DEV)
    y = layer(x)
    ref = O.conv_block_forward(x.cpu(), O.gate_weights(layer.weights.detach().cpu(), True, torch.float32), sel, (1, 1), (1, 1), (3, 3))
    assert (y.detach().cpu() - ref).abs().max().item() <= 1e-5


def test_flatten_hands_over_to_packed_logic_layers():
    torch.manual_seed(9)
    n, c, h, w = 150, 4, 6, 6
    bits = torch.randint(0, 2, (n, c, h, w), device=DEV).bool()
    p = C.PackBitsTensor(bits, 64)
    flat = torch.nn.Flatten()(p)
    assert flat is p and not p.image
    ref = C.PackBitsTensor(bits.flatten(1), 64)
    assert p.pad_len == ref.pad_len and torch.equal(p.t, ref.t)
    fc = C.LogicLayer(c * h * w, 80, implementation="cuda").to(DEV).eval()
    counts = C.GroupSum(4)(fc(p))
    want = C.GroupSum(4)(fc(C.PackBitsTensor(bits.flatten(1), 64)))
    assert torch.equal(counts, want) and counts.shape == (n, 4)


def test_packed_block_errors():
    layer = _layer(3, 4, 1, 1, 3, seed=0)
    bits = torch.randint(0, 2, (10, 3, 8, 8), device=DEV).bool()
    with pytest.raises(ValueError):
        C.PackBitsTensor(bits, 32)
    with pytest.raises(AssertionError):
        layer(C.PackBitsTensor(bits.flatten(1), 64))        # not an image batch
    with pytest.raises(AssertionError):
        layer.train()(C.PackBitsTensor(bits, 64))
    layer.eval()
    x = C.PackBitsTensor(bits, 64).t
    gates = layer.weights.argmax(-1).to(torch.uint8)
    with pytest.raises(RuntimeError):
        convlogic_hip.full_convlogic_eval_packed(x.int(), gates, layer.selection, 1, 1, 1, 1, 3, 3)
    with pytest.raises(RuntimeError):
        convlogic_hip.full_convlogic_eval_packed(x, gates[:, :4].contiguous(), layer.selection, 1, 1, 1, 1, 3, 3)
    with pytest.raises(RuntimeError, match="divisible by 2"):
        convlogic_hip.full_convlogic_eval_packed(x[:, :, :7].contiguous(), gates, layer.selection, 1, 1, 1, 1, 3, 3)


@pytest.mark.parametrize("samples,cin,cout", [(2048, 6, 9), (2100, 24, 40), (4160, 16, 33), (8192, 12, 21)])
def test_packed_block_4x4_one_group_per_lane(samples, cin, cout, monkeypatch):
    # from 32 word groups on, 4x4 images take the kernels that give every lane one group of 64 samples (full blocks of
    # 64 groups: two passes of 32 samples with planes fetched by the wavefront together; the rest of the batch: one
    # 64-bit pass): against the numpy oracle (bit-exact), against the staged kernel and the 64-bit pass alone, with a
    # ragged last wavefront and last word, and with kernels that read more than two channels
    torch.manual_seed(samples + cin)
    ch = torch.randint(0, cin, (cout, 2))
    pick = torch.randint(0, 2, (cout, 8))
    chan = torch.gather(ch, 1, pick)
    chan[1] = torch.arange(8) % cin                                  # up to eight channels
    chan[cout - 1, 5] = (chan[cout - 1, 0] + 1) % cin
    chan[cout - 1, 6] = (chan[cout - 1, 0] + 2) % cin
    sel = ((chan << 16) | (torch.randint(0, 3, (cout, 8)) << 8) | torch.randint(0, 3, (cout, 8))).to(torch.int32)
    layer = _layer(cin, cout, 1, 1, 3, seed=3, selection=sel.to(DEV))
    bits = torch.randint(0, 2, (samples, cin, 4, 4), device=DEV).bool()
    gates = layer.weights.argmax(-1).to(torch.uint8)
    words, pad = O.pack_image(bits.cpu().numpy())
    want = O.conv_block_eval_packed(words, gates.cpu().numpy(), sel.numpy(), (1, 1), (1, 1), (3, 3))
    p = layer(C.PackBitsTensor(bits, 64))
    assert p.pad_len == pad and np.array_equal(p.t.cpu().numpy(), want)
    x_words = torch.from_numpy(words).to(DEV)
    set_knobs(monkeypatch, CLG_FWD_4X4="0")
    staged = convlogic_hip.full_convlogic_eval_packed(x_words, gates, layer.selection, 1, 1, 1, 1, 3, 3)
    set_knobs(monkeypatch, CLG_FWD_4X4=None)
    assert torch.equal(staged, p.t)
    set_knobs(monkeypatch, CLG_PACKED_4X4_HALVES="0")
    whole = convlogic_hip.full_convlogic_eval_packed(x_words, gates, layer.selection, 1, 1, 1, 1, 3, 3)
    assert torch.equal(whole, p.t)


@pytest.mark.parametrize("samples,cin,cout", [(2048, 6, 9), (4160, 16, 33), (8192, 12, 21), (1000, 6, 9)])
def test_packed_block_4x4_feature_major_output(samples, cin, cout):
    # the last block can write its words [C, 2, 2, G]: the same words as the [G, C, 2, 2] kernels, flatten() then takes a
    # view instead of a transpose, and the packed LogicLayer behind it gives the same result; batches below 32 groups
    # (the 1000-sample case) keep the group-major kernels and the transpose
    torch.manual_seed(samples + cout)
    layer = _layer(cin, cout, 1, 1, 3, seed=5)
    bits = torch.randint(0, 2, (samples, cin, 4, 4), device=DEV).bool()
    gates = layer.weights.argmax(-1).to(torch.uint8)
    x_words = C.PackBitsTensor(bits, 64).t
    plain = convlogic_hip.full_convlogic_eval_packed(x_words, gates, layer.selection, 1, 1, 1, 1, 3, 3)
    fm = convlogic_hip.full_convlogic_eval_packed(x_words, gates, layer.selection, 1, 1, 1, 1, 3, 3, feature_major=True)
    groups = x_words.shape[0]
    assert fm.shape == plain.shape and torch.equal(fm, plain)
    assert fm.is_contiguous() == (groups < 32) and (groups < 32 or fm.permute(1, 2, 3, 0).is_contiguous())
    head = C.LogicLayer(cout * 4, cout * 8, implementation="cuda").to(DEV).eval()
    outs = []
    for flag in (False, True):
        layer.feature_major_output = flag
        p = layer(C.PackBitsTensor(bits, 64))
        before = p.t.data_ptr()
        p.flatten()
        assert p.t.shape == (cout * 4, groups) and p.t.is_contiguous() and not p.image
        assert (p.t.data_ptr() == before) == (flag and groups >= 32)           # a view of the block's output, or a transposed copy
        outs.append(head(p).t.clone())
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("n,cin,cout,hw", [(70, 128, 24, 8), (5, 6, 9, 4), (33, 40, 16, 2), (3, 3, 8, 16)])
def test_one_position_per_lane_equals_two_rows_per_lane(n, cin, cout, hw, monkeypatch):
    # workgroups whose samples fill at most half a wavefront with (row pair, column) slots give every conv position
    # its own lane and pool across lanes; same bits and same float values (pooling choice included) as the default
    # mapping, and the packed result against the oracle
    set_knobs(monkeypatch, CLG_FWD_4X4="0")
    layer = _layer(cin, cout, 1, 1, 3, seed=n)
    bits = torch.randint(0, 2, (n * 64, cin, hw, hw), device=DEV).bool() if n <= 5 else torch.randint(0, 2, (n, cin, hw, hw), device=DEV).bool()
    gates = layer.weights.argmax(-1).to(torch.uint8)
    words, pad = O.pack_image(bits.cpu().numpy())
    x_words = torch.from_numpy(words).to(DEV)
    x = torch.rand(n, cin, hw, hw, device=DEV)
    wp = torch.softmax(layer.weights.detach(), -1)
    got = {}
    for mode in ("1", "0"):
        set_knobs(monkeypatch, CLG_FWD_ONE_ROW=mode)                   # 0: every shape keeps two rows per lane
        got[mode] = (convlogic_hip.full_convlogic_eval_packed(x_words, gates, layer.selection, 1, 1, 1, 1, 3, 3),
                     *convlogic_hip.full_convlogic_forward(x, wp, layer.selection, 1, 1, 1, 1, 3, 3))
    for a, b in zip(got["1"], got["0"]):
        assert torch.equal(a, b)
    want = O.conv_block_eval_packed(words, gates.cpu().numpy(), layer.selection.cpu().numpy(), (1, 1), (1, 1), (3, 3))
    assert np.array_equal(got["1"][0].cpu().numpy(), want)

"""GPU parity of the packed-bit path (pack, bitwise evaluation, per-class counts): bit-exact against
the numpy oracle; the reference holds no tests for this path, so the oracle itself is pinned by
closed forms only (tests/test_oracle.py)."""
import numpy as np
import pytest
import torch

import convlogic_amd as C
from convlogic_amd.hip import _lib, difflogic_hip
from oracle import convlogic_oracle as O
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu
TORCH_WORD = {8: torch.int8, 16: torch.int16, 32: torch.int32, 64: torch.int64}


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
@pytest.mark.parametrize("batch,features", [(1, 1), (7, 3), (64, 5), (100, 130), (129, 257), (1000, 33), (4096, 16), (70, 48),
                                            (257, 1024), (64, 4112), (5, 32),
                                            # 8..15 and >= 16 groups of 64 samples with 16 | features: the LDS-transposing kernels,
                                            # ragged last group, last word and last feature tile
                                            (1000, 48), (600, 160), (1030, 32), (520, 4112), (2049, 528)])
def test_pack_bits_both_layouts(bits, batch, features):
    rng = np.random.default_rng(batch * 7 + features)
    t = rng.integers(0, 2, (batch, features)).astype(bool)
    want, pad = O.pack_bits(t.T, bits)
    tt = torch.from_numpy(t).to(DEV)
    w1, p1 = difflogic_hip.tensor_packbits_cuda(tt.T.contiguous(), bits)
    w2, p2 = difflogic_hip.tensor_packbits_sample_major(tt, bits)
    assert p1 == p2 == pad and w1.dtype == TORCH_WORD[bits]
    assert np.array_equal(w1.cpu().numpy(), want) and np.array_equal(w2.cpu().numpy(), want)
    p = C.PackBitsTensor(tt, bits)
    assert p.pad_len == pad and np.array_equal(p.t.cpu().numpy(), want)


@pytest.mark.parametrize("bits,batch", [(64, 4096), (64, 100), (32, 1000), (16, 48), (8, 8), (8, 24), (32, 96)])
def test_eval_packed_bit_exact(bits, batch):
    rng = np.random.default_rng(bits + batch)
    torch.manual_seed(bits + batch)
    in_dim, out_dim = 37, 53
    t = rng.integers(0, 2, (in_dim, batch)).astype(bool)
    words, pad = O.pack_bits(t, bits)
    idx0, idx1 = torch.randint(0, in_dim, (out_dim,)), torch.randint(0, in_dim, (out_dim,))
    gate = (torch.arange(out_dim) % 16).to(torch.uint8)
    want = O.eval_packed(words, idx0.numpy(), idx1.numpy(), gate.numpy())
    got = difflogic_hip.eval(torch.from_numpy(words).to(DEV), idx0.to(DEV), idx1.to(DEV), gate.to(DEV))
    assert got.dtype == TORCH_WORD[bits] and np.array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("bits,batch,features,k", [(64, 256, 40, 10), (32, 100, 12, 3), (8, 9, 4, 2), (64, 5000, 2000, 10), (16, 33, 6, 6),
                                                   (64, 4133, 84, 4), (32, 4200, 30, 3), (8, 600, 9, 1), (64, 8192, 2400, 4),
                                                   (64, 4096, 7, 7), (64, 4096, 40000, 2)])
def test_group_bit_sum(bits, batch, features, k):
    rng = np.random.default_rng(batch + features)
    t = rng.integers(0, 2, (features, batch)).astype(bool)
    words, pad = O.pack_bits(t, bits)
    got = difflogic_hip.groupbitsum(torch.from_numpy(words).to(DEV), pad, k)
    want = O.group_bit_sum(words, pad, k)
    assert got.dtype == torch.int32 and got.shape == (batch, k) and np.array_equal(got.cpu().numpy(), want)


def test_packed_stack_equals_float_eval_path():
    # 3 LogicLayers + GroupSum in eval mode: packed bits vs the float path on the same binary input
    torch.manual_seed(3)
    dims = [96, 192, 160, 120]
    layers = [C.LogicLayer(a, b, implementation="cuda") for a, b in zip(dims[:-1], dims[1:])]
    model = torch.nn.Sequential(*layers, C.GroupSum(10, tau=6.5)).to(DEV).eval()
    x = torch.randint(0, 2, (300, dims[0]), device=DEV).bool()
    with torch.no_grad():
        y_float = model(x.float())
        y_bits = model(C.PackBitsTensor(x, 64))
    assert y_bits.dtype == torch.int32 and y_bits.shape == (300, 10)
    assert torch.equal(y_bits.float() / 6.5, y_float)
    # and against the oracle, bit for bit, layer by layer
    words, pad = O.pack_bits(x.cpu().numpy().T, 64)
    for layer in layers:
        words = O.eval_packed(words, layer.indices_0.cpu().numpy(), layer.indices_1.cpu().numpy(),
                              layer.weights.argmax(-1).cpu().numpy().astype(np.uint8))
    assert np.array_equal(O.group_bit_sum(words, pad, 10), y_bits.cpu().numpy())


def test_eval_packed_config2_row_shape_properties():
    # BASELINE config 2 row shape (1024 int64 words per feature) with fewer features; bit-exact vs oracle
    rng = np.random.default_rng(9)
    torch.manual_seed(9)
    in_dim = out_dim = 2000
    words = rng.integers(-2**63, 2**63 - 1, (in_dim, 1024), dtype=np.int64)
    layer = C.LogicLayer(in_dim, out_dim, implementation="cuda").to(DEV).eval()
    gate = layer.weights.argmax(-1).to(torch.uint8)
    got = difflogic_hip.eval(torch.from_numpy(words).to(DEV), layer.indices_0, layer.indices_1, gate)
    want = O.eval_packed(words, layer.indices_0.cpu().numpy(), layer.indices_1.cpu().numpy(), gate.cpu().numpy())
    assert np.array_equal(got.cpu().numpy(), want)
    # De Morgan: evaluating the complemented gates on complemented inputs complements the output
    comp = torch.tensor([15 - ((g & 8) >> 3 | (g & 4) >> 1 | (g & 2) << 1 | (g & 1) << 3) for g in range(16)], dtype=torch.uint8, device=DEV)
    got_c = difflogic_hip.eval(~torch.from_numpy(words).to(DEV), layer.indices_0, layer.indices_1, comp[gate.long()])
    assert torch.equal(~got_c, got)


def test_eval_packed_config2_full_size_properties():
    # BASELINE config 2 at full size: 64000 -> 64000 neurons, 65536 samples in 1024 int64 words per feature (524 MB per
    # tensor), through the module path (walk-ordered kernel).  Checked by properties the size does not change:
    # pass-through gates reproduce the wired input rows (against torch's own gather), the walk-ordered kernel equals
    # the plain one on random gates, and complemented gates on complemented inputs complement the output.
    torch.manual_seed(2)
    width, words = 64000, 1024
    x = torch.randint(-2**63, 2**63 - 1, (width, words), dtype=torch.int64, device=DEV)
    layer = C.LogicLayer(width, width, implementation="cuda").to(DEV).eval()
    packed = C.PackBitsTensor.__new__(C.PackBitsTensor)
    packed.bit_count, packed.pad_len, packed.t = 64, 0, x
    with torch.no_grad():
        layer.weights.zero_()
        layer.weights[: width // 2, 3] = 1.0                        # gate 3: A
        layer.weights[width // 2:, 5] = 1.0                         # gate 5: B
        out = layer(packed).t
        assert torch.equal(out[: width // 2], x[layer.indices_0[: width // 2]])
        assert torch.equal(out[width // 2:], x[layer.indices_1[width // 2:]])
        del out
        layer.weights.copy_(torch.randn_like(layer.weights))
        gate = layer.weights.argmax(-1).to(torch.uint8)
        packed.t = x
        walked = layer(packed).t
        plain = difflogic_hip.eval(x, layer.indices_0, layer.indices_1, gate)
        assert torch.equal(walked, plain)
        del plain
        comp = torch.tensor([15 - ((g & 8) >> 3 | (g & 4) >> 1 | (g & 2) << 1 | (g & 1) << 3) for g in range(16)],
                            dtype=torch.uint8, device=DEV)
        got_c = difflogic_hip.eval(~x, layer.indices_0, layer.indices_1, comp[gate.long()])
        assert torch.equal(~got_c, walked)
        # per-class counts of the full tensor: every sample's ten counts sum to the number of set bits in its column
        counts = difflogic_hip.groupbitsum(walked, 0, 10)
        assert counts.shape == (65536, 10) and int(counts.sum().item()) == _popcount_sum(walked)


def _popcount_sum(words):
    """number of set bits of an int64 tensor, on the GPU, 16 bits at a time through a lookup table"""
    table = torch.tensor([bin(i).count("1") for i in range(65536)], dtype=torch.int64, device=words.device)
    total = 0
    for shift in (0, 16, 32, 48):
        total += int(table[((words >> shift) & 0xFFFF)].sum().item())
    return total


def test_packed_errors():
    x = torch.zeros(8, 4, dtype=torch.bool, device=DEV)
    with pytest.raises(ValueError):
        difflogic_hip.tensor_packbits_cuda(x, 12)
    p = C.PackBitsTensor(x.T.contiguous(), 32)
    with pytest.raises(ValueError):
        p.group_sum(3)
    with pytest.raises(NotImplementedError):
        C.PackBitsTensor(torch.zeros(4, 4, dtype=torch.bool))
    layer = C.LogicLayer(8, 8, implementation="cuda").to(DEV)
    with pytest.raises(AssertionError):
        layer(p)                       # training mode
    assert p.flatten() is p


@pytest.mark.parametrize("in_dim,out_dim,words,bits", [(37, 53, 128, 64), (64, 64, 1024, 64), (500, 300, 200, 64), (20, 100, 130, 64),
                                                         (16, 16, 512, 32), (9, 30, 64, 64), (300, 150, 256, 64)])
def test_eval_planned_equals_unplanned(in_dim, out_dim, words, bits):
    # the walk-ordered kernel must give the bits of the plain kernel and of the oracle for any wiring,
    # including neurons wired twice to one feature and features used once
    rng = np.random.default_rng(in_dim + words)
    torch.manual_seed(in_dim + words)
    info = np.iinfo(O.NP_WORD[bits])
    x = rng.integers(info.min, info.max, (in_dim, words), dtype=O.NP_WORD[bits])
    if out_dim * 2 >= in_dim and in_dim != 20:
        layer = C.LogicLayer(in_dim, out_dim, implementation="python")
        idx0, idx1 = layer.indices_0, layer.indices_1
    else:
        idx0, idx1 = torch.randint(0, in_dim, (out_dim,)), torch.randint(0, in_dim, (out_dim,))
        idx1[:7] = idx0[:7]
    gate = torch.randint(0, 16, (out_dim,), dtype=torch.uint8)
    xd, a, b, g = torch.from_numpy(x).to(DEV), idx0.to(DEV), idx1.to(DEV), gate.to(DEV)
    plan = difflogic_hip.eval_plan(a, b, in_dim)
    assert sorted((plan.cpu() & 0x0FFFFFFF).tolist()) == list(range(out_dim))
    got = difflogic_hip.eval_planned(xd, a, b, g, plan)
    assert torch.equal(got, difflogic_hip.eval(xd, a, b, g))
    assert np.array_equal(got.cpu().numpy(), O.eval_packed(x, idx0.numpy(), idx1.numpy(), gate.numpy()))


@pytest.mark.parametrize("in_dim,out_dim,words,bits", [(64, 96, 1024, 64), (37, 53, 128, 64), (16, 40, 512, 32), (9, 30, 64, 64)])
def test_eval_planned_from_logits_takes_the_gates_torch_argmax_takes(in_dim, out_dim, words, bits):
    # arg-max inside the evaluation kernel (rows of at least 1 KiB) or by the separate launch (the 512-byte rows of the
    # last case): in both cases the gate ids of torch.argmax -- first maximum on ties, -0 == +0, a NaN beats everything,
    # the first NaN wins -- and the bits of the oracle
    rng = np.random.default_rng(in_dim * 7 + words)
    torch.manual_seed(in_dim * 7 + words)
    info = np.iinfo(O.NP_WORD[bits])
    x = rng.integers(info.min, info.max, (in_dim, words), dtype=O.NP_WORD[bits])
    idx0, idx1 = torch.randint(0, in_dim, (out_dim,)), torch.randint(0, in_dim, (out_dim,))
    logits = torch.randn(out_dim, 16)
    logits[0] = 0.0                                                  # all equal: gate 0
    logits[1, 3] = logits[1, 9] = 7.0                                # tie: the first
    logits[2] = -1.0
    logits[2, 5], logits[2, 11] = -0.0, 0.0                          # -0 and +0 tie: the first
    logits[3, 2], logits[3, 6] = float("inf"), float("nan")         # NaN above +inf
    logits[4, 10], logits[4, 12] = float("nan"), float("nan")       # the first NaN
    logits[5] = float("-inf")
    logits[6, 15] = 100.0
    logits[7] = -torch.arange(16.0) * 1e-30                          # denormal steps downwards: gate 0
    want = logits.argmax(-1)
    assert want[:8].tolist() == [0, 3, 5, 6, 10, 0, 15, 0]
    xd, a, b, lg = torch.from_numpy(x).to(DEV), idx0.to(DEV), idx1.to(DEV), logits.to(DEV)
    plan = difflogic_hip.eval_plan(a, b, in_dim)
    got = difflogic_hip.eval_planned_logits(xd, a, b, lg, plan)
    assert torch.equal(got, difflogic_hip.eval_planned(xd, a, b, difflogic_hip.gate_argmax(lg), plan))
    assert np.array_equal(got.cpu().numpy(), O.eval_packed(x, idx0.numpy(), idx1.numpy(), want.numpy().astype(np.uint8)))
    # float64 logits: the two-launch route, same result
    assert torch.equal(got, difflogic_hip.eval_planned_logits(xd, a, b, lg.double(), plan))


def test_eval_planned_logits_entry_point_rejects_rows_the_walk_kernel_does_not_take():
    lib = _lib.load()
    x = torch.zeros(8, 16, dtype=torch.int64, device=DEV)            # 128-byte rows
    y = torch.empty(8, 16, dtype=torch.int64, device=DEV)
    a = torch.zeros(8, dtype=torch.int64, device=DEV)
    lg = torch.zeros(8, 16, device=DEV)
    plan = torch.arange(8, dtype=torch.int32, device=DEV)
    assert lib.clg_fc_eval_walk_fits(8, x.data_ptr(), y.data_ptr(), 16) == 0
    assert lib.clg_fc_eval_walk_fits(8, x.data_ptr(), y.data_ptr(), 128) == 1
    rc = lib.clg_fc_eval_packed_planned_logits(8, x.data_ptr(), a.data_ptr(), a.data_ptr(), lg.data_ptr(), plan.data_ptr(), y.data_ptr(),
                                               8, 8, 16, 0)
    assert rc != 0 and b"clg_fc_eval_walk_fits" in lib.clg_last_error()


def test_eval_plan_follows_in_place_rewiring():
    torch.manual_seed(4)
    layer = C.LogicLayer(40, 60, implementation="cuda").to(DEV).eval()
    bits = torch.randint(0, 2, (2048, 40), device=DEV).bool()
    y1 = layer(C.PackBitsTensor(bits, 64)).t.clone()
    layer.indices_0.copy_(torch.randint(0, 40, (60,), device=DEV))      # as the reference tests rewire a layer
    y2 = layer(C.PackBitsTensor(bits, 64)).t
    words, _ = O.pack_bits(bits.cpu().numpy().T, 64)
    want = O.eval_packed(words, layer.indices_0.cpu().numpy(), layer.indices_1.cpu().numpy(),
                         layer.weights.argmax(-1).cpu().numpy().astype(np.uint8))
    assert np.array_equal(y2.cpu().numpy(), want) and not torch.equal(y1, y2)


@pytest.mark.timeout(600)
def test_eval_packed_config2_full_size_vs_c_oracle():
    # BASELINE config 2 at full size against the CPU oracle, word for word: 3 layers of 64000 neurons on 65536 samples in
    # 1024 int64 words per feature through the module path, every layer's output compared with oracle/packed_oracle.c
    # (OpenMP, about 25 ms per layer on the host cores), then the per-class counts against numpy on the oracle's words.
    import ctypes
    import os
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "libpacked_oracle.so")
    if not os.path.exists(path):
        pytest.skip("oracle/libpacked_oracle.so not built (make -C oracle)")
    lib = ctypes.CDLL(path)
    width, words, k = 64000, 1024, 10
    rng = np.random.default_rng(22)
    x = rng.integers(-2**63, 2**63 - 1, (width, words), dtype=np.int64, endpoint=True)
    torch.manual_seed(22)
    layers = [C.LogicLayer(width, width, implementation="cuda").to(DEV).eval() for _ in range(3)]
    packed = C.PackBitsTensor.__new__(C.PackBitsTensor)
    packed.bit_count, packed.pad_len, packed.image, packed.t = 64, 0, False, torch.from_numpy(x).to(DEV)
    ref = x
    vp = ctypes.c_void_p
    with torch.no_grad():
        for i, layer in enumerate(layers):
            packed = layer(packed)
            a = layer.indices_0.cpu().numpy().astype(np.int64)
            b = layer.indices_1.cpu().numpy().astype(np.int64)
            gate = layer.weights.argmax(-1).cpu().numpy().astype(np.uint8)
            out = np.empty_like(ref)
            lib.oracle_eval_packed(ref.ctypes.data_as(vp), a.ctypes.data_as(vp), b.ctypes.data_as(vp), gate.ctypes.data_as(vp),
                                   out.ctypes.data_as(vp), ctypes.c_int64(width), ctypes.c_int64(words * 8))
            assert np.array_equal(packed.t.cpu().numpy(), out), f"layer {i}"
            ref = out
        counts = packed.group_sum(k).cpu().numpy()
    assert counts.shape == (65536, k) and counts.dtype == np.int32
    per = width // k
    for g in range(k):                                               # class g: rows g*per .. (g+1)*per, sample s = bit s%8 of byte s/8
        bits = np.unpackbits(ref[g * per:(g + 1) * per].view(np.uint8), axis=1, bitorder="little")
        assert np.array_equal(counts[:, g], bits.sum(axis=0, dtype=np.int32)), f"class {g}"


def test_eval_packed_walk_with_eight_vectors_per_lane(monkeypatch):
    # the walk-ordered kernel keeps 4 vectors of a row per lane by default; 8 is the variant a knob selects: same words
    from tests.gpu_util import set_knobs
    torch.manual_seed(4)
    layer = C.LogicLayer(120, 200, implementation="cuda").to(DEV).eval()
    x = torch.randint(0, 2, (70000, 120), device=DEV).bool()         # rows of 1094 words: more than one 8 KiB chunk, ragged
    outs = []
    for r in (None, "8", "4"):
        set_knobs(monkeypatch, CLG_EVAL_WALK_R=r)
        with torch.no_grad():
            outs.append(layer(C.PackBitsTensor(x, 64)).t.clone())
    set_knobs(monkeypatch, CLG_EVAL_WALK_R=None)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    words, pad = O.pack_bits(x.cpu().numpy().T, 64)
    want = O.eval_packed(words, layer.indices_0.cpu().numpy(), layer.indices_1.cpu().numpy(), layer.weights.argmax(-1).cpu().numpy().astype(np.uint8))
    assert np.array_equal(outs[1].cpu().numpy(), want)

"""Pins the CPU oracle (oracle/) before anything is compared against it.

Every check here is independent of the oracle's own formula: truth tables from the
bits of the gate id, the reference's known-answer tests, brute force on tiny inputs,
library routines (torch max_pool2d, numpy packbits) and golden wiring vectors written
from the reference constructors.
"""
import ctypes
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import convlogic_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def truth(i, a, b):
    """bit of gate id i for inputs (a,b): id = f00*8 + f01*4 + f10*2 + f11."""
    return (i >> (3 - (2 * a + b))) & 1


# ---- the 16 ops -------------------------------------------------------------
@pytest.mark.parametrize("i", range(16))
def test_bin_op_truth_table(i):
    for a in (0, 1):
        for b in (0, 1):
            got = O.bin_op(torch.tensor([float(a)]), torch.tensor([float(b)]), i)
            assert got.item() == truth(i, a, b)


@pytest.mark.parametrize("i", range(16))
def test_bin_op_is_multilinear_extension(i):
    # the relaxation must be the unique multilinear interpolant of the truth table
    a, b = torch.rand(50, dtype=torch.float64), torch.rand(50, dtype=torch.float64)
    want = sum(truth(i, p, q) * (a if p else 1 - a) * (b if q else 1 - b) for p in (0, 1) for q in (0, 1))
    assert torch.allclose(O.bin_op(a, b, i), want, atol=1e-14)


def test_bin_op_eval_bitwise_truth_table():
    for i in range(16):
        for a in (0, 1):
            for b in (0, 1):
                wa = np.array([-1 if a else 0], dtype=np.int64)
                wb = np.array([-1 if b else 0], dtype=np.int64)
                got = O.bin_op_eval(wa, wb, i)[0]
                assert got == (-1 if truth(i, a, b) else 0)


def test_anf_identity():
    # y = m0 ^ (m1&a) ^ (m2&b) ^ (m3&a&b) with masks from the truth table
    rng = np.random.default_rng(0)
    a = rng.integers(-2**63, 2**63 - 1, 64, dtype=np.int64)
    b = rng.integers(-2**63, 2**63 - 1, 64, dtype=np.int64)
    for i in range(16):
        f00, f01, f10, f11 = truth(i, 0, 0), truth(i, 0, 1), truth(i, 1, 0), truth(i, 1, 1)
        m = [np.int64(-1 if v else 0) for v in (f00, f00 ^ f10, f00 ^ f01, f00 ^ f01 ^ f10 ^ f11)]
        anf = m[0] ^ (m[1] & a) ^ (m[2] & b) ^ (m[3] & a & b)
        assert np.array_equal(anf, O.bin_op_eval(a, b, i))


def test_coef_matrix_matches_truth_tables():
    # c_1=f00, c_a=f10-f00, c_b=f01-f00, c_ab=f00-f01-f10+f11
    for i in range(16):
        f00, f01, f10, f11 = truth(i, 0, 0), truth(i, 0, 1), truth(i, 1, 0), truth(i, 1, 1)
        assert O.COEF[:, i].tolist() == [f00 - f01 - f10 + f11, f10 - f00, f01 - f00, f00]


def test_fold_equals_16_term_sum():
    torch.manual_seed(0)
    w = torch.softmax(torch.randn(7, 16, dtype=torch.float64), -1)
    a, b = torch.rand(7, dtype=torch.float64), torch.rand(7, dtype=torch.float64)
    c = O.fold_coefficients(w)
    assert torch.allclose(c[:, 0] * a * b + c[:, 1] * a + c[:, 2] * b + c[:, 3], O.bin_op_s(a, b, w), atol=1e-14)


# ---- reference known-answer tests --------------------------------------------
def test_kat_all_gates_logic_layer():
    # tests/difflogic/test_difflogic_forward.py:74-100 (training mode, -inf logits, exact)
    idx0 = torch.tensor([0, 2, 4, 6]).repeat(16)
    idx1 = torch.tensor([1, 3, 5, 7]).repeat(16)
    logits = torch.full((64, 16), float("-inf"))
    for g in range(16):
        logits[g * 4: g * 4 + 4, g] = 0.0
    flat = [0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0]
    y = O.logic_fc_forward(torch.tensor([flat]), idx0, idx1, O.gate_weights(logits, True))
    want = torch.tensor([[float(truth(g, int(flat[2 * s]), int(flat[2 * s + 1]))) for g in range(16) for s in range(4)]])
    assert torch.equal(y, want)


def test_kat_all_gates_tree():
    # tests/convlogic/test_treelogic_forward.py:66-86
    logits = torch.full((16, 4, 16), float("-inf"))
    for g in range(16):
        logits[g, :, g] = 0.0
    flat = [0.0, 0.0, 0.0, 1.0, 1.0, 0.0, 1.0, 1.0]
    x = torch.tensor(flat).reshape(1, 1, 1, 1, 8).expand(-1, 16, -1, -1, -1)
    y = O.tree_forward(x, O.gate_weights(logits, True))
    want = torch.tensor([[float(truth(g, int(flat[2 * s]), int(flat[2 * s + 1]))) for s in range(4)] for g in range(16)])
    assert torch.equal(y.view(16, 4), want)


def test_residual_init_probability():
    w = torch.zeros(16)
    w[3] = 5.0
    assert abs(torch.softmax(w, -1)[3].item() - np.exp(5) / (np.exp(5) + 15)) < 1e-6


# ---- fully connected ----------------------------------------------------------
def test_fc_forward_vs_loops():
    torch.manual_seed(1)
    x = torch.rand(3, 6, dtype=torch.float64)
    idx0, idx1 = torch.randint(0, 6, (9,)), torch.randint(0, 6, (9,))
    w = torch.softmax(torch.randn(9, 16, dtype=torch.float64), -1)
    assert torch.allclose(O.logic_fc_forward(x, idx0, idx1, w), O.logic_fc_forward_loops(x, idx0, idx1, w), atol=1e-14)


def test_fc_gradcheck():
    torch.manual_seed(2)
    x = torch.rand(4, 5, dtype=torch.float64, requires_grad=True)
    logits = torch.randn(7, 16, dtype=torch.float64, requires_grad=True)
    idx0, idx1 = torch.randint(0, 5, (7,)), torch.randint(0, 5, (7,))
    assert torch.autograd.gradcheck(lambda a, l: O.logic_fc_forward(a, idx0, idx1, torch.softmax(l, -1)), (x, logits),
                                    eps=1e-6, atol=1e-4)


def test_csr_brute_force():
    torch.manual_seed(3)
    idx0, idx1 = torch.randint(0, 7, (11,)), torch.randint(0, 7, (11,))
    start, flat = O.csr_build(idx0, idx1, 7)
    assert start[0] == 0 and start[-1] == 22 and len(flat) == 22
    for i in range(7):
        want = sorted([y for y in range(11) if idx0[y] == i] + [y for y in range(11) if idx1[y] == i])
        assert sorted(flat[start[i]: start[i + 1]].tolist()) == want


def test_group_sum():
    x = torch.arange(12.0).view(1, 12)
    assert torch.equal(O.group_sum(x, 3, 2.0), torch.tensor([[3.0, 11.0, 19.0]]))


# ---- wiring: golden vectors from the reference constructors -------------------
def test_connections_golden(golden):
    for rec in golden["logic_layer"]:
        torch.manual_seed(rec["seed"])
        w = torch.randn(rec["out_dim"], 16)          # the constructor draws the logits first
        assert abs(float(w.double().sum()) - rec["weights_sum"]) < 1e-9
        fn = O.random_connections if rec["connections"] == "random" else O.unique_connections
        a, b = fn(rec["in_dim"], rec["out_dim"])
        assert a.tolist() == rec["indices_0"] and b.tolist() == rec["indices_1"]


def test_selection_golden(golden):
    for rec in golden["conv_layer"]:
        torch.manual_seed(rec["seed"])
        k = rec["kernel"]
        k = (k, k) if isinstance(k, int) else tuple(k)
        w = torch.randn(rec["out_channels"], 7 if rec["complete"] else 4, 16)
        assert abs(float(w.double().sum()) - rec["weights_sum"]) < 1e-9
        sel = O.generate_selection(rec["in_channels"], rec["out_channels"], k, rec["groups"])
        assert sel.tolist() == rec["selection"]


def test_selection_invariants():
    torch.manual_seed(7)
    sel = O.generate_selection(9, 64, (3, 3))
    ch, ry, rx = O.unpack_selection(sel)
    assert int(ch.max()) < 9 and int(ry.max()) < 3 and int(rx.max()) < 3
    for c in range(64):
        assert len(set(ch[c].tolist())) <= 2
        for p in range(4):
            assert sel[c, 2 * p] != sel[c, 2 * p + 1]


# ---- conv ---------------------------------------------------------------------
@pytest.mark.parametrize("stride,pad,kernel", [((1, 1), (1, 1), (3, 3)), ((2, 2), (2, 2), (4, 4)), ((1, 2), (0, 1), (2, 3))])
def test_conv4_vectorised_vs_loops(stride, pad, kernel):
    torch.manual_seed(4)
    x = torch.randn(2, 3, 7, 8, dtype=torch.float64)
    sel = O.generate_selection(3, 4, kernel)
    w = torch.softmax(torch.randn(4, 4, 16, dtype=torch.float64), -1)
    a = O.conv4_forward(x, w, sel, stride, pad, kernel)
    b = O.conv4_forward_loops(x, w, sel, stride, pad, kernel)
    assert a.shape == b.shape and torch.allclose(a, b, atol=1e-14)


def test_conv_block_is_split_pipeline_and_pool():
    torch.manual_seed(5)
    x = torch.randn(2, 3, 10, 10)
    sel = O.generate_selection(3, 2, (3, 3))
    w = torch.softmax(torch.randn(2, 7, 16), -1)
    y, x2, x3, idx = O.conv_block_forward(x, w, sel, (1, 1), (1, 1), (3, 3), return_all=True)
    assert x2.shape == (2, 2, 10, 10, 4) and x3.shape == (2, 2, 10, 10, 2) and y.shape == (2, 2, 5, 5)
    x4 = O.tree_forward(x3, w[:, 6:7]).squeeze(-1)
    # strict '>' running max in window order (0,0),(0,1),(1,0),(1,1): brute force
    for n in range(2):
        for c in range(2):
            for py in range(5):
                for px in range(5):
                    best, bi = -float("inf"), -1
                    for dy in range(2):
                        for dx in range(2):
                            v = x4[n, c, 2 * py + dy, 2 * px + dx].item()
                            if v > best:
                                best, bi = v, (2 * py + dy) * 10 + 2 * px + dx
                    assert y[n, c, py, px].item() == best and idx[n, c, py * 5 + px].item() == bi


def test_pool_tie_rule_first_max():
    x = torch.zeros(1, 1, 4, 4)
    _, idx = F.max_pool2d(x, 2, 2, return_indices=True)
    assert idx.flatten().tolist() == [0, 2, 8, 10]


def test_conv_block_eval_binary_is_binary():
    torch.manual_seed(6)
    x = torch.randint(0, 2, (2, 2, 6, 6)).float()
    sel = O.generate_selection(2, 3, (3, 3))
    w = O.gate_weights(torch.randn(3, 7, 16), False)
    y = O.conv_block_forward(x, w, sel, (1, 1), (1, 1), (3, 3))
    assert torch.all((y == 0) | (y == 1))


def test_conv_block_gradcheck():
    torch.manual_seed(8)
    x = torch.rand(2, 2, 6, 6, dtype=torch.float64, requires_grad=True)
    logits = torch.randn(3, 7, 16, dtype=torch.float64, requires_grad=True)
    sel = O.generate_selection(2, 3, (3, 3))
    fn = lambda a, l: O.conv_block_forward(a, torch.softmax(l, -1), sel, (1, 1), (1, 1), (3, 3))
    assert torch.autograd.gradcheck(fn, (x, logits), eps=1e-6, atol=1e-4)


# ---- packed bits ---------------------------------------------------------------
@pytest.mark.parametrize("bits", [8, 16, 32, 64])
@pytest.mark.parametrize("b", [1, 7, 64, 100, 129])
def test_pack_bits_vs_loops(bits, b):
    rng = np.random.default_rng(b)
    t = rng.integers(0, 2, (5, b)).astype(bool)
    w1, p1 = O.pack_bits(t, bits)
    w2, p2 = O.pack_bits_loops(t, bits)
    assert p1 == p2 == (bits - b % bits) % bits and w1.dtype == w2.dtype and np.array_equal(w1, w2)
    assert np.array_equal(O.unpack_bits(w1, p1), t)


def test_eval_packed_vs_float_path():
    # unpack -> float eval path on {0,1} (exact) -> compare bits
    rng = np.random.default_rng(1)
    torch.manual_seed(1)
    f, b, out = 10, 200, 24
    t = rng.integers(0, 2, (f, b)).astype(bool)
    words, pad = O.pack_bits(t, 64)
    idx0, idx1 = torch.randint(0, f, (out,)), torch.randint(0, f, (out,))
    logits = torch.randn(out, 16)
    gate = logits.argmax(-1).numpy().astype(np.uint8)
    y_bits = O.unpack_bits(O.eval_packed(words, idx0.numpy(), idx1.numpy(), gate), pad)
    y_float = O.logic_fc_forward(torch.from_numpy(t.T.astype(np.float32)), idx0, idx1, O.gate_weights(logits, False))
    assert np.array_equal(y_bits, y_float.numpy().T.astype(bool))


def test_group_bit_sum_closed_form():
    rng = np.random.default_rng(2)
    t = rng.integers(0, 2, (12, 70)).astype(bool)
    words, pad = O.pack_bits(t, 32)
    got = O.group_bit_sum(words, pad, 3)
    want = t.reshape(3, 4, 70).sum(1).T
    assert got.dtype == np.int32 and got.shape == (70, 3) and np.array_equal(got, want)


def _c_oracle():
    path = os.path.join(ROOT, "oracle", "libpacked_oracle.so")
    if not os.path.exists(path):
        pytest.skip("oracle/libpacked_oracle.so not built (make -C oracle)")
    return ctypes.CDLL(path)


@pytest.mark.parametrize("bits", [8, 16, 32, 64])
def test_c_oracle_matches_numpy_oracle(bits):
    lib = _c_oracle()
    rng = np.random.default_rng(bits)
    f, b, out, k = 12, 300, 18, 3
    t = rng.integers(0, 2, (f, b)).astype(np.uint8)
    words, pad = O.pack_bits(t.astype(bool), bits)
    cw = np.zeros_like(words)
    lib.oracle_pack_bits(t.ctypes.data_as(ctypes.c_void_p), cw.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(f),
                         ctypes.c_int64(b), ctypes.c_int(bits))
    assert np.array_equal(cw, words)
    idx0 = rng.integers(0, f, out).astype(np.int64)
    idx1 = rng.integers(0, f, out).astype(np.int64)
    gate = (np.arange(out) % 16).astype(np.uint8)
    y = np.zeros((out, words.shape[1]), dtype=words.dtype)
    row_bytes = words.shape[1] * words.itemsize
    lib.oracle_eval_packed(words.ctypes.data_as(ctypes.c_void_p), idx0.ctypes.data_as(ctypes.c_void_p),
                           idx1.ctypes.data_as(ctypes.c_void_p), gate.ctypes.data_as(ctypes.c_void_p),
                           y.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(out), ctypes.c_int64(row_bytes))
    assert np.array_equal(y, O.eval_packed(words, idx0, idx1, gate))
    gs = np.zeros((words.shape[1] * bits - pad, k), dtype=np.int32)
    lib.oracle_group_bit_sum(y.ctypes.data_as(ctypes.c_void_p), gs.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(out),
                             ctypes.c_int64(row_bytes), ctypes.c_int64(pad), ctypes.c_int64(k))
    assert np.array_equal(gs, O.group_bit_sum(y, pad, k))


# ---- packed conv block -----------------------------------------------------------------------------
def test_pack_image_round_trip_and_bit_positions():
    rng = np.random.default_rng(3)
    t = rng.integers(0, 2, (130, 2, 3, 5)).astype(bool)
    words, pad = O.pack_image(t)
    assert words.shape == (3, 2, 3, 5) and words.dtype == np.int64 and pad == 62
    assert np.array_equal(O.unpack_image(words, pad), t)
    # sample 64 g + s sits in bit s of group g, straight from the definition
    for n, c, y, x in [(0, 0, 0, 0), (63, 1, 2, 4), (64, 0, 1, 1), (129, 1, 0, 3)]:
        assert ((int(words[n // 64, c, y, x]) >> (n % 64)) & 1) == int(t[n, c, y, x])


@pytest.mark.parametrize("stride,pad,kernel", [(1, 1, 3), (2, 2, 4), (1, 0, 3), ((1, 2), (0, 1), (2, 3))])
def test_conv_block_eval_packed_equals_float_eval_on_bits(stride, pad, kernel):
    # the packed block is DEFINED as the float eval-mode block on {0,1} inputs: compare against the float
    # oracle (itself pinned by the brute-force and max_pool2d tests above) sample by sample
    pr = lambda v: (v, v) if isinstance(v, int) else tuple(v)
    stride, pad, kernel = pr(stride), pr(pad), pr(kernel)
    torch.manual_seed(11)
    n, cin, c, h, w = 70, 3, 5, 9, 11
    ho, wo = O.conv_out_size(h, w, stride, pad, kernel)
    h += (ho % 2) * stride[0]
    w += (wo % 2) * stride[1]
    sel = O.generate_selection(cin, c, kernel)
    logits = torch.randn(c, 7, 16)
    bits = torch.randint(0, 2, (n, cin, h, w)).bool()
    want = O.conv_block_forward(bits.float(), O.gate_weights(logits, False, torch.float32), sel, stride, pad, kernel)
    assert torch.all((want == 0) | (want == 1))
    words, pad_len = O.pack_image(bits.numpy())
    got = O.conv_block_eval_packed(words, logits.argmax(-1).numpy().astype(np.uint8), sel.numpy(), stride, pad, kernel)
    assert np.array_equal(O.unpack_image(got, pad_len), want.numpy() > 0.5)


def test_conv_block_eval_packed_all_gates_truth_table():
    # one kernel, 1x1 taps on a 2x2 image of constants: root gate id i over leaves that pass tap 0 / tap 1
    # through (gate 3 = A) must reproduce bit (3 - 2a - b) of i -- the truth-table rule of the gate ids
    sel = torch.tensor([[(0 << 16), (1 << 16), (0 << 16), (1 << 16), (1 << 16), (0 << 16), (1 << 16), (0 << 16)]], dtype=torch.int32)
    for i in range(16):
        gates = np.array([[3, 3, 3, 3, 3, 3, i]], dtype=np.uint8)      # leaves: taps 0,2,4,6; middles pass leaf 0 / leaf 2
        for a in (0, 1):
            for b in (0, 1):
                img = np.zeros((1, 2, 2, 2), dtype=np.int64)
                img[:, 0], img[:, 1] = -a, -b                           # all 64 samples set or clear
                y = O.conv_block_eval_packed(img, gates, sel.numpy(), (1, 1), (0, 0), (1, 1))
                assert y.shape == (1, 1, 1, 1) and int(y[0, 0, 0, 0]) == -((i >> (3 - 2 * a - b)) & 1), (i, a, b)


# ---- input binarisation --------------------------------------------------------------------------
def test_thresholds_closed_forms():
    assert torch.allclose(O.thresholds_uniform(3), torch.tensor([0.25, 0.5, 0.75]))          # BASELINE config 4: linspace(1,3,3)/4
    assert torch.allclose(O.thresholds_uniform(1), torch.tensor([0.5]))
    x = torch.arange(100, dtype=torch.float32).flip(0) / 100                                  # sorted: 0.00 .. 0.99
    assert torch.allclose(O.thresholds_distributive(x, 3), torch.tensor([0.25, 0.50, 0.75]))  # index floor(100 i / 4)
    assert torch.allclose(O.thresholds_distributive(x, 1), torch.tensor([0.50]))


def test_apply_thresholds_is_threshold_major_and_strict():
    img = torch.tensor([[[0.25, 0.3]], [[0.5, 0.9]]])                                         # [C=2, 1, 2]
    out = O.apply_thresholds(img, torch.tensor([0.25, 0.5, 0.75]))
    assert out.shape == (6, 1, 2)
    # channel l*C + c; the comparison is strict (0.25 > 0.25 is false)
    assert out[:, 0].tolist() == [[0.0, 1.0], [1.0, 1.0], [0.0, 0.0], [0.0, 1.0], [0.0, 0.0], [0.0, 1.0]]
    batch = torch.rand(5, 2, 3, 4)
    got = O.apply_thresholds(batch, torch.tensor([0.3, 0.6]))
    for n in range(5):
        assert torch.equal(got[n], O.apply_thresholds(batch[n], torch.tensor([0.3, 0.6])))

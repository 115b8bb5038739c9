"""CPU oracle for the logic-layer hot path.  TEST INFRASTRUCTURE ONLY.

This file restates, on the CPU with torch / numpy, the algorithm of the
reference's python path (and, where the reference has only a CUDA kernel, the
semantics of that kernel).  It is imported only by tests/, by
__graft_entry__.smoke() and by bench.py's cpu_baseline leg -- never by the
product package (convlogic_amd), which must fail loudly when its HIP library
is missing.

Each function cites the reference file:line it follows (paths relative to the
reference checkout).  How each function is pinned (see tests/test_oracle.py):

  function                    pinned by
  --------------------------  -------------------------------------------------
  bin_op / bin_op_s           truth table of gate id bits; reference KATs
                              (tests/difflogic/test_difflogic_forward.py:74-100,
                              tests/convlogic/test_treelogic_forward.py:66-86)
  fold_coefficients           equality with the 16-term sum on random inputs;
                              COEF matrix of difflogic_kernel.cu:164-167
  logic_fc_forward            brute-force python loops on tiny sizes
  csr_build                   brute force
  random/unique connections,  golden vectors written from the reference
  generate_selection          constructors (tests/golden/wiring_golden.json)
  conv4_forward (vectorised)  literal nested-loop restatement on tiny sizes;
                              closed form iy = oy*sh + ry - ph
  tree_forward                reference KAT (all 16 gates, exact)
  conv_block_forward          composition + torch max_pool2d (library routine,
                              tie -> first max in row-major window order)
  gradients                   torch autograd over the restated forward +
                              float64 gradcheck
  pack_bits                   numpy.packbits(bitorder="little") vs per-bit loop
  eval_packed                 bitwise truth table brute-forced over 16x4; ANF
                              identity; unpack -> float eval -> repack
  group_bit_sum               unpack + reshape-sum
                              (the reference has NO tests for the packed path:
                              pack_bits / eval_packed / group_bit_sum are
                              "parity unpinned by the reference" and pinned
                              only by the closed forms above)
  pack_image / unpack_image   round trip; bit positions read from the definition
  conv_block_eval_packed      no reference counterpart (new capability): defined
                              as conv_block_forward in eval mode on {0,1} inputs
                              and checked against it sample by sample; 16-gate
                              truth-table test
  thresholds_*,               closed forms: linspace(1,L,L)/(L+1); quantile
  apply_thresholds            indices on a known ramp; strict ">" and the
                              threshold-major channel order on a written-out image
"""
import numpy as np
import torch
import torch.nn.functional as F

# rows: coefficient of (a*b, a, b, 1); columns: gate id.  Same integer matrix the
# reference multiplies its four partial sums with
# (src/difflogic/cuda/difflogic_kernel.cu:164-167).
COEF = torch.tensor(
    [[0, 1, -1, 0, -1, 0, -2, -1, 1, 2, 0, 1, 0, 1, -1, 0],
     [0, 0, 1, 1, 0, 0, 1, 1, -1, -1, 0, 0, -1, -1, 0, 0],
     [0, 0, 0, 0, 1, 1, 1, 1, -1, -1, -1, -1, 0, 0, 0, 0],
     [0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 1, 1, 1, 1, 1]], dtype=torch.float64)


# ----------------------------------------------------------------------------
# the 16 relaxed binary operators -- src/difflogic/functional.py:27-71
# ----------------------------------------------------------------------------
def bin_op(a, b, i):
    """Real-valued relaxation of 2-input boolean function number i
    (src/difflogic/functional.py:27-63; table :7-24)."""
    ab = a * b
    if i == 0:
        return torch.zeros_like(a)
    if i == 1:
        return ab
    if i == 2:
        return a - ab
    if i == 3:
        return a
    if i == 4:
        return b - ab
    if i == 5:
        return b
    if i == 6:
        return a + b - 2 * ab
    if i == 7:
        return a + b - ab
    if i == 8:
        return 1 - (a + b - ab)
    if i == 9:
        return 1 - (a + b - 2 * ab)
    if i == 10:
        return 1 - b
    if i == 11:
        return 1 - b + ab
    if i == 12:
        return 1 - a
    if i == 13:
        return 1 - a + ab
    if i == 14:
        return 1 - ab
    if i == 15:
        return torch.ones_like(a)
    raise ValueError(i)


def bin_op_s(a, b, w):
    """r = sum_i w[..., i] * op_i(a, b), accumulated i = 0..15 in order
    (src/difflogic/functional.py:66-71)."""
    r = torch.zeros_like(a)
    for i in range(16):
        r = r + w[..., i] * bin_op(a, b, i)
    return r


def fold_coefficients(w):
    """[..., 16] gate weights -> [..., 4] coefficients (c_ab, c_a, c_b, c_1) with
    sum_i w_i op_i(a,b) == c_ab*a*b + c_a*a + c_b*b + c_1 (every op is multilinear)."""
    return w @ COEF.to(w.dtype).T


def gate_weights(logits, training, dtype=None):
    """softmax in training, one_hot(argmax) in eval
    (src/difflogic/difflogic.py:117-120, src/convlogic/convlogic_layer.py:321-325)."""
    if training:
        return F.softmax(logits, dim=-1)
    return F.one_hot(logits.argmax(-1), 16).to(dtype or logits.dtype)


# ----------------------------------------------------------------------------
# fully connected LogicLayer -- src/difflogic/difflogic.py:112-123
# ----------------------------------------------------------------------------
def logic_fc_forward(x, idx0, idx1, w_prob):
    """x [..., in] -> y [..., out]; neuron j reads x[..., idx0[j]], x[..., idx1[j]]."""
    a, b = x[..., idx0], x[..., idx1]
    return bin_op_s(a, b, w_prob)


def logic_fc_forward_loops(x, idx0, idx1, w_prob):
    """Same as logic_fc_forward with explicit python loops (tiny sizes only)."""
    bsz, out = x.shape[0], len(idx0)
    y = torch.zeros(bsz, out, dtype=x.dtype)
    for n in range(bsz):
        for j in range(out):
            a, b = x[n, int(idx0[j])], x[n, int(idx1[j])]
            acc = torch.zeros((), dtype=x.dtype)
            for i in range(16):
                acc = acc + w_prob[j, i] * bin_op(a, b, i)
            y[n, j] = acc
    return y


def csr_build(idx0, idx1, in_dim):
    """Reverse map input -> neurons that read it (src/difflogic/difflogic.py:71-87):
    for y in order, y is appended to list[idx0[y]] then to list[idx1[y]]."""
    lists = [[] for _ in range(in_dim)]
    for y in range(len(idx0)):
        lists[int(idx0[y])].append(y)
        lists[int(idx1[y])].append(y)
    start = np.array([0] + [len(g) for g in lists]).cumsum()
    flat = [v for g in lists for v in g]
    return torch.tensor(start, dtype=torch.int64), torch.tensor(flat, dtype=torch.int64)


def random_connections(in_dim, out_dim):
    """src/difflogic/difflogic.py:169-181 (consumes the global torch RNG)."""
    assert out_dim * 2 >= in_dim
    c = torch.randperm(2 * out_dim) % in_dim
    c = torch.randperm(in_dim)[c]
    c = c.reshape(2, out_dim)
    return c[0].to(torch.int64), c[1].to(torch.int64)


def unique_connections(in_dim, out_dim):
    """src/difflogic/functional.py:77-125 (consumes the global torch RNG once)."""
    assert out_dim * 2 >= in_dim
    x = torch.arange(in_dim).long().unsqueeze(0)
    a, b = x[..., ::2], x[..., 1::2]
    if a.shape[-1] != b.shape[-1]:
        m = min(a.shape[-1], b.shape[-1])
        a, b = a[..., :m], b[..., :m]
    if a.shape[-1] < out_dim:
        a_, b_ = x[..., 1::2], x[..., 2::2]
        a, b = torch.cat([a, a_], dim=-1), torch.cat([b, b_], dim=-1)
        if a.shape[-1] != b.shape[-1]:
            m = min(a.shape[-1], b.shape[-1])
            a, b = a[..., :m], b[..., :m]
    offset = 2
    while out_dim > a.shape[-1] > offset:
        a_, b_ = x[..., :-offset], x[..., offset:]
        a, b = torch.cat([a, a_], dim=-1), torch.cat([b, b_], dim=-1)
        offset += 1
    if a.shape[-1] < out_dim:
        raise AssertionError((a.shape[-1], offset, out_dim))
    a, b = a[..., :out_dim], b[..., :out_dim]
    perm = torch.randperm(out_dim)
    return a[:, perm].squeeze(0).contiguous(), b[:, perm].squeeze(0).contiguous()


def group_sum(x, k, tau):
    """src/difflogic/difflogic.py:207-208."""
    return x.reshape(*x.shape[:-1], k, x.shape[-1] // k).sum(-1) / tau


# ----------------------------------------------------------------------------
# conv logic -- src/convlogic/convlogic_layer.py
# ----------------------------------------------------------------------------
def unpack_selection(sel):
    """ch<<16 | row<<8 | col (src/convlogic/convlogic_layer.py:175-179)."""
    return (sel >> 16) & 0xFFFF, (sel >> 8) & 0xFF, sel & 0xFF


def generate_selection(in_channels, out_channels, kernel, groups=1, num_inputs=8):
    """src/convlogic/convlogic_layer.py:377-452 (consumes the global torch RNG in the
    same call order: per group randint x2, picks, rows, cols, then conflict re-draws)."""
    kh, kw = kernel
    base, rem = in_channels // groups, in_channels % groups
    sizes = torch.full((groups,), base)
    sizes[:rem] += 1
    starts = torch.cat([torch.zeros(1), sizes.cumsum(0)])[:-1].to(torch.int32)
    all_idx = torch.arange(in_channels, dtype=torch.int32)
    group_map = [all_idx[int(s): int(s) + int(sizes[i])] for i, s in enumerate(starts)]
    out_per = out_channels // groups
    group_ids = torch.clamp(torch.arange(out_channels) // out_per, 0, groups - 1)
    chosen = torch.empty((out_channels, 2), dtype=torch.int32)
    for gid, chans in enumerate(group_map):
        idxs = (group_ids == gid).nonzero(as_tuple=True)[0]
        cnt = idxs.numel()
        if cnt > 0:
            k = chans.numel()
            chosen[idxs, 0] = chans[torch.randint(0, k, (cnt,))]
            chosen[idxs, 1] = chans[torch.randint(0, k, (cnt,))]
    picks = torch.randint(0, 2, (out_channels, num_inputs), dtype=torch.int32)
    ch_sel = torch.where(picks == 0, chosen[:, 0:1].expand(-1, num_inputs), chosen[:, 1:2].expand(-1, num_inputs))
    rows = torch.randint(0, kh, (out_channels, num_inputs), dtype=torch.int32)
    cols = torch.randint(0, kw, (out_channels, num_inputs), dtype=torch.int32)
    for k in range(0, num_inputs, 2):
        conflict = (ch_sel[:, k] == ch_sel[:, k + 1]) & (rows[:, k] == rows[:, k + 1]) & (cols[:, k] == cols[:, k + 1])
        if conflict.any():
            for idx in conflict.nonzero(as_tuple=True)[0].tolist():
                while True:
                    new_r = torch.randint(0, kh, (1,), dtype=torch.int32)
                    new_c = torch.randint(0, kw, (1,), dtype=torch.int32)
                    if not (new_r.item() == rows[idx, k].item() and new_c.item() == cols[idx, k].item()):
                        rows[idx, k + 1] = new_r
                        cols[idx, k + 1] = new_c
                        break
    return (ch_sel << 16) | (rows << 8) | cols


def conv_out_size(h, w, stride, pad, kernel):
    """src/convlogic/convlogic_layer.py:192-193."""
    return (h + 2 * pad[0] - kernel[0]) // stride[0] + 1, (w + 2 * pad[1] - kernel[1]) // stride[1] + 1


def gather_taps(x, sel, stride, pad, kernel):
    """[N,Cin,H,W] -> [N,C,Ho,Wo,8]: tap t of kernel c at (oy,ox) reads
    x[n, ch, oy*sh + ry - ph, ox*sw + rx - pw], zero outside the image
    (src/convlogic/convlogic_layer.py:262-282; full_convlogic_kernel.cu:43-57)."""
    n, _, h, w = x.shape
    ho, wo = conv_out_size(h, w, stride, pad, kernel)
    ch, ry, rx = unpack_selection(sel.long())                       # [C,8]
    xp = F.pad(x, (pad[1], pad[1], pad[0], pad[0]))
    oy = torch.arange(ho).view(1, ho, 1, 1)
    ox = torch.arange(wo).view(1, 1, wo, 1)
    iy = oy * stride[0] + ry.view(-1, 1, 1, 8)                      # padded coords, [C,Ho,1,8]
    ix = ox * stride[1] + rx.view(-1, 1, 1, 8)
    chx = ch.view(-1, 1, 1, 8).expand(-1, ho, wo, 8)
    return xp[:, chx, iy.expand(-1, ho, wo, 8), ix.expand(-1, ho, wo, 8)]


def conv4_forward(x, w_prob4, sel, stride, pad, kernel):
    """Split layer: 4 leaf gates per kernel -> [N,C,Ho,Wo,4]
    (src/convlogic/convlogic_layer.py:181-229)."""
    taps = gather_taps(x, sel, stride, pad, kernel)
    c = sel.shape[0]
    return bin_op_s(taps[..., 0::2], taps[..., 1::2], w_prob4.view(1, c, 1, 1, 4, 16))


def conv4_forward_loops(x, w_prob4, sel, stride, pad, kernel):
    """Literal nested-loop restatement of src/convlogic/convlogic_layer.py:203-229
    (tiny sizes only)."""
    n, _, h, w = x.shape
    c_out = sel.shape[0]
    ho, wo = conv_out_size(h, w, stride, pad, kernel)
    a = x.new_zeros((n, c_out, ho, wo, 4))
    b = x.new_zeros((n, c_out, ho, wo, 4))
    for p in range(4):
        for c in range(c_out):
            s1, s2 = int(sel[c, 2 * p]), int(sel[c, 2 * p + 1])
            ch1, ry1, rx1 = (s1 >> 16) & 0xFFFF, (s1 >> 8) & 0xFF, s1 & 0xFF
            ch2, ry2, rx2 = (s2 >> 16) & 0xFFFF, (s2 >> 8) & 0xFF, s2 & 0xFF
            for oy in range(ho):
                for ox in range(wo):
                    iy1, ix1 = oy * stride[0] + ry1 - pad[0], ox * stride[1] + rx1 - pad[1]
                    iy2, ix2 = oy * stride[0] + ry2 - pad[0], ox * stride[1] + rx2 - pad[1]
                    if 0 <= iy1 < h and 0 <= ix1 < w:
                        a[:, c, oy, ox, p] = x[:, ch1, iy1, ix1]
                    if 0 <= iy2 < h and 0 <= ix2 < w:
                        b[:, c, oy, ox, p] = x[:, ch2, iy2, ix2]
    return bin_op_s(a, b, w_prob4.view(1, c_out, 1, 1, 4, 16))


def tree_forward(x, w_prob):
    """One pairwise level on the last dim: [N,C,H,W,2X] -> [N,C,H,W,X]
    (src/convlogic/treelogic_layer.py:111-127)."""
    c, xo = w_prob.shape[0], w_prob.shape[1]
    return bin_op_s(x[..., 0::2], x[..., 1::2], w_prob.view(1, c, 1, 1, xo, 16))


def conv_block_forward(x, w_prob7, sel, stride, pad, kernel, return_all=False):
    """Fused block = conv4 -> tree(4->2) -> tree(2->1) -> 2x2/2 max-pool
    (src/convlogic/convlogic_layer.py:231-316).  Weight slices 0:4 / 4:6 / 6:7 (:237-239).
    Pool indices are in_y*Wo + in_x in the conv-output plane, first max in window order
    (src/convlogic/cuda/full_convlogic_kernel.cu:135-144)."""
    x2 = conv4_forward(x, w_prob7[:, 0:4], sel, stride, pad, kernel)
    x3 = tree_forward(x2, w_prob7[:, 4:6])
    x4 = tree_forward(x3, w_prob7[:, 6:7]).squeeze(-1)
    y, idx = F.max_pool2d(x4, 2, 2, return_indices=True)
    if return_all:
        return y, x2, x3, idx.flatten(2).to(torch.int32)
    return y


# ----------------------------------------------------------------------------
# packed-bit inference -- src/difflogic/cuda/difflogic_kernel.cu:271-482,
# src/common/cuda_utils.cuh:162-199.  No python twin exists in the reference.
# ----------------------------------------------------------------------------
NP_WORD = {8: np.int8, 16: np.int16, 32: np.int32, 64: np.int64}
NP_UWORD = {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}


def pack_bits(t_fb, bit_count=32):
    """bool [F,B] -> (words [F, ceil(B/bits)], pad_len): bit i of word c is sample
    bits*c + i, LSB first, zero padded (difflogic_kernel.cu:354-362, pad_len :375)."""
    t = np.asarray(t_fb).astype(bool)
    f, b = t.shape
    pad_len = (bit_count - b % bit_count) % bit_count
    tp = np.concatenate([t, np.zeros((f, pad_len), dtype=bool)], axis=1)
    by = np.packbits(tp, axis=1, bitorder="little")                 # [F, (B+pad)/8] uint8
    words = np.ascontiguousarray(by).view("<u%d" % (bit_count // 8)).astype(NP_UWORD[bit_count])
    return words.view(NP_WORD[bit_count]), pad_len


def pack_bits_loops(t_fb, bit_count=32):
    """Per-bit restatement of difflogic_kernel.cu:354-362 (tiny sizes only)."""
    t = np.asarray(t_fb).astype(bool)
    f, b = t.shape
    wn = -(-b // bit_count)
    out = np.zeros((f, wn), dtype=NP_UWORD[bit_count])
    for r in range(f):
        for c in range(wn):
            v = 0
            for i in range(bit_count):
                col = bit_count * c + i
                if col < b and t[r, col]:
                    v |= 1 << i
            out[r, c] = v
    return out.view(NP_WORD[bit_count]), (bit_count - b % bit_count) % bit_count


def bin_op_eval(a, b, op):
    """Bitwise twin of bin_op on packed words (src/common/cuda_utils.cuh:162-199)."""
    if op == 0:
        return np.zeros_like(a)
    if op == 1:
        return a & b
    if op == 2:
        return a & ~b
    if op == 3:
        return a.copy()
    if op == 4:
        return b & ~a
    if op == 5:
        return b.copy()
    if op == 6:
        return a ^ b
    if op == 7:
        return a | b
    if op == 8:
        return ~(a | b)
    if op == 9:
        return ~(a ^ b)
    if op == 10:
        return ~b
    if op == 11:
        return ~b | a
    if op == 12:
        return ~a
    if op == 13:
        return ~a | b
    if op == 14:
        return ~(a & b)
    return ~np.zeros_like(a)


def eval_packed(words, idx0, idx1, gate):
    """y[j] = g_j(x[idx0[j]], x[idx1[j]]) on packed rows (difflogic_kernel.cu:271-293)."""
    words = np.asarray(words)
    idx0, idx1, gate = np.asarray(idx0), np.asarray(idx1), np.asarray(gate)
    out = np.empty((len(idx0), words.shape[1]), dtype=words.dtype)
    a, b = words[idx0], words[idx1]
    for op in range(16):
        m = gate == op
        if m.any():
            out[m] = bin_op_eval(a[m], b[m], op)
    return out


def unpack_bits(words, pad_len=0):
    """inverse of pack_bits -> bool [F, W*bits - pad_len]."""
    words = np.ascontiguousarray(words)
    f = words.shape[0]
    by = words.view(np.uint8).reshape(f, -1)
    bits = np.unpackbits(by, axis=1, bitorder="little").astype(bool)
    return bits[:, : bits.shape[1] - pad_len] if pad_len else bits


def group_bit_sum(words, pad_len, k):
    """int32 [S,k]: out[s,g] = number of set sample-s bits over the F/k features of
    class g; the last pad_len samples are dropped (difflogic_kernel.cu:417-482)."""
    bits = unpack_bits(words, pad_len)                              # [F,S]
    f, s = bits.shape
    assert f % k == 0
    return bits.reshape(k, f // k, s).sum(1).astype(np.int32).T.copy()


def pack_image(t_nchw):
    """bool [N,C,H,W] -> (int64 words [ceil(N/64), C, H, W], pad_len): bit s of group g is sample
    64 g + s (the sample-to-bit rule of difflogic_kernel.cu:354-362 with the group index leading)."""
    t = np.asarray(t_nchw).astype(bool)
    n, c, h, w = t.shape
    words, pad_len = pack_bits(t.reshape(n, c * h * w).T, 64)      # [F, G]
    return np.ascontiguousarray(words.T).reshape(-1, c, h, w), pad_len


def unpack_image(words, pad_len=0):
    """inverse of pack_image -> bool [N,C,H,W]."""
    words = np.asarray(words)
    g, c, h, w = words.shape
    bits = unpack_bits(np.ascontiguousarray(words.reshape(g, c * h * w).T), pad_len)   # [F, N]
    return np.ascontiguousarray(bits.T).reshape(-1, c, h, w)


def conv_block_eval_packed(words, gates, sel, stride, pad, kernel):
    """Packed-bit inference of the fused block on group-major words [G,Cin,H,W] -> [G,C,Ho/2,Wo/2].
    No counterpart in the reference (its packed kernels cover LogicLayer only); defined as its
    eval-mode block (arg-max gates, src/convlogic/convlogic_layer.py:321-325; taps :262-282; tree
    pairs :289-305; 2x2 max pool :316) on {0,1} inputs: every gate becomes its bitwise twin
    (src/common/cuda_utils.cuh:162-199) and the max of bits is their OR."""
    words = np.asarray(words)
    gates = np.asarray(gates)
    g, _, h, w = words.shape
    ho, wo = conv_out_size(h, w, stride, pad, kernel)
    ch, ry, rx = (np.asarray(v) for v in unpack_selection(torch.as_tensor(np.asarray(sel)).long()))   # [C,8]
    c = ch.shape[0]
    xp = np.pad(words, ((0, 0), (0, 0), (pad[0], pad[0]), (pad[1], pad[1])))
    oy = np.arange(ho).reshape(1, ho, 1) * stride[0]
    ox = np.arange(wo).reshape(1, 1, wo) * stride[1]

    def tap(t):
        return xp[:, ch[:, t].reshape(c, 1, 1), oy + ry[:, t].reshape(c, 1, 1), ox + rx[:, t].reshape(c, 1, 1)]   # [G,C,Ho,Wo]

    def level(inputs, first_gate):
        out = []
        for q in range(len(inputs) // 2):
            a, b = inputs[2 * q], inputs[2 * q + 1]
            r = np.empty_like(a)
            for k in range(c):
                r[:, k] = bin_op_eval(a[:, k], b[:, k], int(gates[k, first_gate + q]))
            out.append(r)
        return out

    root = level(level(level([tap(t) for t in range(8)], 0), 4), 6)[0]
    return root[:, :, 0::2, 0::2] | root[:, :, 0::2, 1::2] | root[:, :, 1::2, 0::2] | root[:, :, 1::2, 1::2]


# ----------------------------------------------------------------------------
# input binarisation -- src/convlogic/data.py:46-71
# ----------------------------------------------------------------------------
def thresholds_uniform(levels):
    """src/convlogic/data.py:56-59."""
    return torch.linspace(1, levels, levels, dtype=torch.float32) / (levels + 1)


def thresholds_distributive(x_all, levels):
    """src/convlogic/data.py:62-65."""
    sorted_x = torch.sort(x_all.reshape(-1))[0]
    idx = (sorted_x.shape[0] * torch.arange(1, levels + 1) / (levels + 1)).long()
    return sorted_x[idx]


def apply_thresholds(x, thresholds):
    """One image [C,H,W] -> [L*C,H,W], or a batch [N,C,H,W] -> [N,L*C,H,W]: threshold-major
    concatenation of (x > t) (src/convlogic/data.py:46-50 concatenates along dim 0 of one image)."""
    dim = 0 if x.dim() == 3 else 1
    return torch.cat([(x > t).float() for t in thresholds], dim=dim)

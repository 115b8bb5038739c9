"""Host-side helpers of the logic layers: the 16 relaxed binary operators, wiring generators and
the gradient scaling function.  Interface of the reference's src/difflogic/functional.py."""
import torch

BITS_TO_TORCH_DTYPE = {8: torch.int8, 16: torch.int16, 32: torch.int32, 64: torch.int64}

# Gate i has the truth table (f00, f01, f10, f11) = bits of i, most significant first
# (src/difflogic/functional.py:7-24).  Its real-valued relaxation is the multilinear polynomial
#   f00 + (f10 - f00) a + (f01 - f00) b + (f00 - f01 - f10 + f11) ab.
# GATE_POLY[i] = (c_1, c_a, c_b, c_ab).
GATE_POLY = tuple(
    (f00, f10 - f00, f01 - f00, f00 - f01 - f10 + f11)
    for f00, f01, f10, f11 in (((i >> 3) & 1, (i >> 2) & 1, (i >> 1) & 1, i & 1) for i in range(16))
)


def bin_op(a, b, i):
    """op_i(a, b) for gate id i in 0..15 (src/difflogic/functional.py:27-63)."""
    if not 0 <= i < 16:
        raise ValueError(f"gate id must be in 0..15, got {i}")
    assert a.shape == b.shape, (a.shape, b.shape)
    c1, ca, cb, cab = GATE_POLY[i]
    out = torch.full_like(a, float(c1))
    if ca:
        out = out + ca * a
    if cb:
        out = out + cb * b
    if cab:
        out = out + cab * (a * b)
    return out


def bin_op_s(a, b, i_s):
    """sum_i i_s[..., i] * op_i(a, b) (src/difflogic/functional.py:66-71), evaluated through the
    folded form c_1 + c_a a + c_b b + c_ab ab."""
    poly = torch.tensor(GATE_POLY, dtype=i_s.dtype, device=i_s.device)      # [16, 4]
    coef = i_s @ poly                                                       # [..., 4]
    return coef[..., 0] + coef[..., 1] * a + coef[..., 2] * b + coef[..., 3] * (a * b)


def get_unique_connections(in_dim, out_dim):
    """Wiring in which neighbouring inputs are paired first, then pairs at growing distance, and
    the neurons are shuffled (src/difflogic/functional.py:77-125).  Returns int64 (a, b)."""
    assert out_dim * 2 >= in_dim, (
        f"The number of neurons ({out_dim}) must not be smaller than half of the number of inputs "
        f"({in_dim}) because otherwise not all inputs could be used or considered.")
    idx = torch.arange(in_dim, dtype=torch.int64)

    def pairs(first, second):
        m = min(len(first), len(second))
        return first[:m], second[:m]

    a, b = pairs(idx[0::2], idx[1::2])                       # (0,1), (2,3), ...
    if len(a) < out_dim:                                     # (1,2), (3,4), ...
        a2, b2 = idx[1::2], idx[2::2]
        a, b = pairs(torch.cat([a, a2]), torch.cat([b, b2]))
    offset = 2
    while out_dim > len(a) > offset:                         # (i, i+offset) for offset = 2, 3, ...
        a, b = torch.cat([a, idx[:-offset]]), torch.cat([b, idx[offset:]])
        offset += 1
    if len(a) < out_dim:
        raise AssertionError((len(a), offset, out_dim))
    perm = torch.randperm(out_dim)
    return a[:out_dim][perm].contiguous(), b[:out_dim][perm].contiguous()


class GradFactor(torch.autograd.Function):
    """Identity whose gradient is scaled by f (src/difflogic/functional.py:131-139)."""

    @staticmethod
    def forward(ctx, x, f):
        ctx.f = f
        return x

    @staticmethod
    def backward(ctx, grad_y):
        return grad_y * ctx.f, None

"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

from oracle import convlogic_oracle as O

DEV = "cuda"


def set_knobs(monkeypatch, **knobs):
    """Sets (value) or removes (None) CLG_* environment knobs and makes the library read them again."""
    from convlogic_amd.hip import _lib
    for name, value in knobs.items():
        if value is None:
            monkeypatch.delenv(name, raising=False)
        else:
            monkeypatch.setenv(name, str(value))
    _lib.reload_knobs()


def has_gpu():
    return torch.cuda.is_available()


def assert_grad_close(got, ref, rel=1e-4, name="grad", rel_elem=None):
    """Gradient parity, three bounds that all must hold:
      (1) global:      ||got - ref||_2 <= rel * ||ref||_2
      (2) per element: |got - ref| <= rel * (|ref| + eps) with eps = the mean magnitude of ref -- the relative
          error |d| / (|ref| + eps) of every element, where eps keeps elements that cancel to (almost) zero from
          being held to rel times nothing
      (3) per element against the LARGEST magnitude: |got - ref| <= rel * (|ref| + max|ref|) (implied by (2) for
          tensors whose mean and maximum are close; kept because it is the bound a single wild element breaks first).
    rel_elem: bound (2) alone may be given a wider value (whole-network tests, where float32 rounding compounds
    through the layers)."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    scale = ref.abs().max().item() + 1e-30
    eps = ref.abs().mean().item() + 1e-30
    err = (got - ref).abs()
    assert (err <= rel * (ref.abs() + scale)).all(), f"{name}: max abs err {err.max().item():.3e}, scale {scale:.3e}"
    worst = (err / (ref.abs() + eps)).max().item()
    assert worst <= (rel if rel_elem is None else rel_elem), f"{name}: per-element relative error {worst:.3e} (eps = mean|ref| = {eps:.3e})"
    l2 = (got - ref).norm().item() / (ref.norm().item() + 1e-30)
    assert l2 <= rel, f"{name}: relative L2 error {l2:.3e}"


def block_oracle(x, logits, sel, stride, pad, kernel, idx_gpu, training=True):
    """Oracle forward of the fused block on the CPU.  Returns (y routed through the GPU's pooling
    choice, oracle pooled y, oracle indices, x2, x3, logits leaf, x leaf) so that gradients can be taken
    along exactly the route the GPU took; near-tie cells where the routes differ are checked by the
    caller."""
    xl = x.detach().cpu().clone().requires_grad_(True)
    ll = logits.detach().cpu().clone().requires_grad_(True)
    w = O.gate_weights(ll, training, xl.dtype)
    y, x2, x3, idx = O.conv_block_forward(xl, w, sel.cpu(), stride, pad, kernel, return_all=True)
    x4 = O.tree_forward(x3, w[:, 6:7]).squeeze(-1)
    routed = x4.flatten(2).gather(2, idx_gpu.cpu().long()).view_as(y)
    return routed, y, idx, x2, x3, ll, xl, x4


def check_pool_route(idx_gpu, idx_ref, x4, tol=1e-5):
    """Where the GPU picked another window position than the oracle, the two values must be within tol
    (a near tie between different tap patterns).  Returns the number of such cells."""
    idx_gpu, idx_ref = idx_gpu.cpu().long(), idx_ref.cpu().long()
    diff = idx_gpu != idx_ref
    if diff.any():
        flat = x4.detach().flatten(2)
        gap = (flat.gather(2, idx_gpu) - flat.gather(2, idx_ref)).abs()
        assert gap[diff].max().item() <= tol, f"pool route differs with gap {gap[diff].max().item():.3e}"
    return int(diff.sum())


def np_i64(t):
    return t.detach().cpu().numpy().astype(np.int64)

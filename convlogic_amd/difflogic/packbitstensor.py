"""PackBitsTensor: eval-only container of bit-packed activations, one sample per bit.
Interface of the reference's src/difflogic/packbitstensor.py."""
import numpy as np
import torch

from ..hip import difflogic_hip


class PackBitsTensor:
    """t: bool [batch, features] on the GPU -> self.t integer words [features, ceil(batch/bit_count)]
    (bit i of word c = sample bit_count*c + i), self.pad_len unused high bits of the last word
    (src/difflogic/packbitstensor.py:11-21)."""

    def __init__(self, t: torch.Tensor, bit_count=32):
        assert len(t.shape) == 2, t.shape
        self.bit_count = bit_count
        if not t.is_cuda:
            raise NotImplementedError(f"PackBitsTensor only supports CUDA tensors, but got {t.device}.")
        # packs straight from the sample-major tensor (no transposed bool copy)
        self.t, self.pad_len = difflogic_hip.tensor_packbits_sample_major(t.contiguous(), self.bit_count)

    @property
    def is_cuda(self):
        return self.t.is_cuda

    @property
    def device(self):
        return self.t.device

    def group_sum(self, k):
        """int32 [batch, k] per-class counts of set bits (src/difflogic/packbitstensor.py:23-24)."""
        return difflogic_hip.groupbitsum(self.t, self.pad_len, k)

    def flatten(self, start_dim=0, end_dim=-1, **kwargs):
        """nn.Flatten is a no-op on packed activations (src/difflogic/packbitstensor.py:26-31)."""
        return self

    def _row_repr(self, row):
        def bits(v):
            return np.binary_repr(int(v), width=self.bit_count)[::-1]
        if len(row) <= 4:
            return " ".join(bits(v) for v in row)
        return " ".join(bits(v) for v in row[:3]) + " ... " + bits(row[-1])

    def __repr__(self):
        return "\n".join(self._row_repr(row) for row in self.t.cpu())

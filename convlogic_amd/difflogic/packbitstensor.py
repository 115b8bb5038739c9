"""PackBitsTensor: eval-only container of bit-packed activations, one sample per bit.
Interface of the reference's src/difflogic/packbitstensor.py."""
import numpy as np
import torch

from ..hip import difflogic_hip


class PackBitsTensor:
    """t: bool [batch, features] on the GPU -> self.t integer words [features, ceil(batch/bit_count)]
    (bit i of word c = sample bit_count*c + i), self.pad_len unused high bits of the last word
    (src/difflogic/packbitstensor.py:11-21).

    Beyond the reference: a 4-D bool image batch [batch, C, H, W] (bit_count 64 only) is kept
    group-major, self.t int64 [ceil(batch/64), C, H, W] with self.image True -- the layout the packed
    conv-logic block reads and writes; flatten() (what nn.Flatten calls) turns it into the
    feature-major layout above with features in c*H*W + y*W + x order."""

    def __init__(self, t: torch.Tensor, bit_count=32):
        assert len(t.shape) in (2, 4), t.shape
        self.bit_count = bit_count
        self.image = False
        if not t.is_cuda:
            raise NotImplementedError(f"PackBitsTensor only supports CUDA tensors, but got {t.device}.")
        if t.dim() == 4:
            if bit_count != 64:
                raise ValueError(f"image batches are packed 64 samples per word, got bit_count={bit_count}")
            n, c, h, w = t.shape
            words, self.pad_len = difflogic_hip.tensor_packbits_sample_major(t.contiguous().view(n, c * h * w), 64)
            self.t = difflogic_hip.transpose(words).view(-1, c, h, w)
            self.image = True
            return
        # packs straight from the sample-major tensor (no transposed bool copy)
        self.t, self.pad_len = difflogic_hip.tensor_packbits_sample_major(t.contiguous(), self.bit_count)

    @classmethod
    def from_image_words(cls, words: torch.Tensor, pad_len: int):
        """Wraps group-major packed image words int64 [groups, C, H, W] (64 samples per word)."""
        assert words.dim() == 4 and words.dtype == torch.int64, (words.shape, words.dtype)
        self = cls.__new__(cls)
        self.t, self.pad_len, self.bit_count, self.image = words, int(pad_len), 64, True
        return self

    @property
    def is_cuda(self):
        return self.t.is_cuda

    @property
    def device(self):
        return self.t.device

    def group_sum(self, k):
        """int32 [batch, k] per-class counts of set bits (src/difflogic/packbitstensor.py:23-24)."""
        if self.image:
            self.flatten()
        return difflogic_hip.groupbitsum(self.t, self.pad_len, k)

    def flatten(self, start_dim=0, end_dim=-1, **kwargs):
        """nn.Flatten is a no-op on feature-major packed activations (src/difflogic/packbitstensor.py:26-31);
        a group-major image batch becomes feature-major here (one 8-byte transpose, or a view when the last
        block already wrote its words feature-major)."""
        if self.image:
            groups = self.t.shape[0]
            by_feature = self.t.permute(*range(1, self.t.dim()), 0)
            if by_feature.is_contiguous():                           # a block that wrote [C, H, W, G]: already feature-major
                self.t = by_feature.reshape(-1, groups)
            else:
                self.t = difflogic_hip.transpose(self.t.reshape(groups, -1))
            self.image = False
        return self

    def _row_repr(self, row):
        def bits(v):
            return np.binary_repr(int(v), width=self.bit_count)[::-1]
        if len(row) <= 4:
            return " ".join(bits(v) for v in row)
        return " ".join(bits(v) for v in row[:3]) + " ... " + bits(row[-1])

    def __repr__(self):
        rows = self.t.reshape(self.t.shape[0], -1).t() if self.image else self.t
        return "\n".join(self._row_repr(row) for row in rows.cpu())

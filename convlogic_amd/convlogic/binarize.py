"""Input binarisation of the reference's data module (src/convlogic/data.py:46-71) as batch functions:
threshold values, the threshold-major {0,1} channel expansion for training, and the same expansion
written straight into packed words for inference."""
import torch

from ..difflogic.packbitstensor import PackBitsTensor
from ..hip import convlogic_hip


def uniform_thresholds(levels: int) -> torch.Tensor:
    """i / (levels + 1) for i = 1..levels, float32 (src/convlogic/data.py:56-59)."""
    return torch.linspace(1, levels, levels, dtype=torch.float32) / (levels + 1)


def distributive_thresholds(x_all: torch.Tensor, levels: int) -> torch.Tensor:
    """Values at the i/(levels+1) positions of the sorted pixels, i = 1..levels (src/convlogic/data.py:62-65)."""
    ordered = torch.sort(x_all.reshape(-1))[0]
    at = (ordered.shape[0] * torch.arange(1, levels + 1) / (levels + 1)).long()
    return ordered[at.to(ordered.device)]


def compute_thresholds(x_all: torch.Tensor, threshold_type: str, levels: int) -> torch.Tensor:
    kind = threshold_type.lower()
    if kind == "uniform":
        return uniform_thresholds(levels)
    if kind == "distributive":
        return distributive_thresholds(x_all, levels)
    raise ValueError(f"Unknown threshold_type: {threshold_type}")


def apply_thresholds(x: torch.Tensor, thresholds: torch.Tensor) -> torch.Tensor:
    """[N, C, H, W] (or one image [C, H, W]) -> float {0,1} with levels*C channels, threshold-major
    (src/convlogic/data.py:46-50).  GPU tensors go through the HIP kernel; host tensors (the data-loader
    side, as in the reference) use the same torch expression as the reference."""
    if x.dim() == 3:
        return apply_thresholds(x.unsqueeze(0), thresholds).squeeze(0)
    if not x.is_cuda:
        return torch.cat([(x > t).float() for t in thresholds], dim=1)
    return convlogic_hip.threshold_images(x.float().contiguous(), thresholds.to(x.device, torch.float32).contiguous())


def pack_thresholds(x: torch.Tensor, thresholds: torch.Tensor) -> PackBitsTensor:
    """GPU images [N, C, H, W] -> PackBitsTensor image batch with levels*C channels, 64 samples per word:
    thresholding and bit packing in one pass over the pixels."""
    if not x.is_cuda:
        raise NotImplementedError(f"pack_thresholds only supports GPU tensors, but got {x.device}.")
    words, pad_len = convlogic_hip.threshold_pack_images(x.float().contiguous(),
                                                         thresholds.to(x.device, torch.float32).contiguous())
    return PackBitsTensor.from_image_words(words, pad_len)

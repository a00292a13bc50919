"""Small helpers with the names the reference exposes (src/triton_gated_mlp/utils.py:27-56)."""

import torch
from torch import Tensor, nn


def copy_weights(model_src: nn.Module, model_tgt: nn.Module) -> None:
    """Copy parameters of model_src into model_tgt, pairing them by registration order and name."""
    for (name_src, p_src), (name_tgt, p_tgt) in zip(model_src.named_parameters(), model_tgt.named_parameters()):
        if name_src == name_tgt:
            p_tgt.data = p_src.data.clone()


def validate_contiguous(x: Tensor) -> Tensor:
    """x itself when it is contiguous, otherwise a contiguous copy."""
    return x if x.is_contiguous() else x.contiguous()


def validate_tensor_device(x: Tensor) -> None:
    """The fused operators take GPU tensors only (there is no interpreter or CPU path here)."""
    if not x.is_cuda:
        raise RuntimeError(f"tensor is on {x.device}: the fused gated-MLP operators need a GPU tensor")


def is_cuda_available() -> bool:
    return torch.cuda.is_available()


def is_cuda() -> bool:
    return torch.cuda.is_available()


def get_device() -> torch.device:
    """`cuda` (the ROCm device in a PyTorch-ROCm build) when a GPU is visible, else `cpu`."""
    return torch.device("cuda" if torch.cuda.is_available() else "cpu")

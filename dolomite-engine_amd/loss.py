"""Side channel for the router's auxiliary loss (lm_engine/hf_models/loss.py:93-116)."""

import torch


_AUX_LOSS: torch.Tensor | float = 0


def clear_aux_loss() -> None:
    global _AUX_LOSS
    _AUX_LOSS = 0


def add_aux_loss(aux_loss: torch.Tensor | float) -> None:
    global _AUX_LOSS
    # (the first layer's loss is taken as it is: 0 + tensor would be a kernel launch for nothing)
    _AUX_LOSS = aux_loss if is_aux_loss_zero(_AUX_LOSS) else _AUX_LOSS + aux_loss


def get_aux_loss() -> torch.Tensor | float:
    return _AUX_LOSS


def is_aux_loss_zero(aux_loss: torch.Tensor | float | None) -> bool:
    if aux_loss is None:
        return True
    if isinstance(aux_loss, torch.Tensor):
        return False
    return aux_loss == 0

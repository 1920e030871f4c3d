"""Import of reference checkpoints into models built from this package.

The reference's training driver leaves `runs/<run>/final.pth` = {'args', 'model_state', 'final_score', ...}
(train.py:295-320) and rebuilds a model by constructing it, replaying the surgery, then `load_state_dict(model_state)`
(utils.py:580-672).  The layers here keep the reference's parameter names and shapes (`experts.w1 [E,D,Ed]`,
`experts.b1 [E,Ed]`, `experts.w2 [E,Ed,D]`, `last_bias [1,D]`, `router.layers.{0,2}.weight`), so a reference
`model_state` loads unchanged once the MoE layers and routers have been installed (`replace_with_moes`, `add_routers`).

Files are read with `torch.load(..., weights_only=True)` only: nothing stored in the file is executed.  A `final.pth`
whose `args` entry is an arbitrary Python object is refused by that loader; re-save its `model_state` alone
(`torch.save({'model_state': state}, path)`) in the environment that wrote it.
"""
from __future__ import annotations

from typing import Dict, Iterable, Tuple

import torch
from torch import nn

from .layer import MoeficationMoE

# prefixes that wrappers add in front of every key: DataParallel / accelerate, torch.compile
WRAPPER_PREFIXES = ('module.', '_orig_mod.')


def read_model_state(path, map_location='cpu') -> Dict[str, torch.Tensor]:
    """The `model_state` of a reference `final.pth` (or a bare state dict), tensors only."""
    try:
        blob = torch.load(path, map_location=map_location, weights_only=True)
    except Exception as exc:  # the safe loader names what it refused
        raise ValueError(f'{path}: not loadable with weights_only=True ({exc}); '
                         "re-save the state dict alone: torch.save({'model_state': state}, path)") from exc
    state = blob.get('model_state', blob) if isinstance(blob, dict) else None
    if not isinstance(state, dict) or not all(isinstance(v, torch.Tensor) for v in state.values()):
        raise ValueError(f'{path}: expected a state dict or a dict with a "model_state" entry')
    return strip_wrapper_prefixes(state)


def strip_wrapper_prefixes(state: Dict[str, torch.Tensor], prefixes: Iterable[str] = WRAPPER_PREFIXES) -> Dict[str, torch.Tensor]:
    """Removes, repeatedly, a prefix that EVERY key carries (what wrapping the model in another module leaves)."""
    state = dict(state)
    changed = True
    while changed and state:
        changed = False
        for pre in prefixes:
            if all(k.startswith(pre) for k in state):
                state = {k[len(pre):]: v for k, v in state.items()}
                changed = True
    return state


def load_model_state(model: nn.Module, state: Dict[str, torch.Tensor], strict: bool = True) -> Tuple[list, list]:
    """`model.load_state_dict` with the shape checks spelled out for the MoE parameters: returns (missing, unexpected)
    key lists (both empty under strict=True, which raises otherwise)."""
    own = model.state_dict()
    for key, value in state.items():
        if key in own and tuple(own[key].shape) != tuple(value.shape):
            raise ValueError(f'{key}: checkpoint shape {tuple(value.shape)} != model shape {tuple(own[key].shape)} '
                             '(was the model converted with the same number of experts / expert size?)')
    result = model.load_state_dict(state, strict=strict)
    return list(result.missing_keys), list(result.unexpected_keys)


def prepack(model: nn.Module) -> int:
    """Builds the MFMA-ordered weight buffers of every MoE layer now (they are otherwise built by the first forward);
    returns the number of bytes they hold.  The model must already sit on its ROCm device in its inference dtype."""
    total = 0
    for module in model.modules():
        if isinstance(module, MoeficationMoE):
            packed = module.packed_weights()
            if packed is not None:
                total += packed.numel() * packed.element_size()
    return total

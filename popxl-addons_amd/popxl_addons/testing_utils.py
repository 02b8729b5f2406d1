"""Eager counterpart of the reference's test harness (popxl_addons/testing_utils.py:25-107): run a
layer on the GPU with numpy inputs and return numpy outputs."""
from typing import Callable, List, Optional

import numpy as np


class TensorInput:
    """Marks a numpy array as a tensor argument of the module (testing_utils.py:19-31)."""

    def __init__(self, data: np.ndarray, dtype=None) -> None:
        self.data = data
        self.dtype = dtype


def run_module(module, *args, weights: Optional[Callable] = None, device="cuda:0", **kwargs) -> List[np.ndarray]:
    """Build the module's variables from the arguments, write `weights` (a mapping, or a callable
    taking the variables) into them, run it and return the outputs as numpy arrays."""
    import torch

    def typed_arg(a):
        if isinstance(a, TensorInput):
            t = torch.from_numpy(np.ascontiguousarray(a.data))
            if a.dtype is not None:
                t = t.to(a.dtype)
            return t.to(device)
        return a

    new_args = [typed_arg(a) for a in args]
    new_kwargs = {k: typed_arg(v) for k, v in kwargs.items()}
    first = next(a for a in new_args if isinstance(a, torch.Tensor))
    if getattr(module, "variables", None) is None:
        module.init_variables(first.shape[-1], first.dtype, first.device)
    if weights is not None:
        module.load_weights(weights)
    outputs = module.build(*new_args, **new_kwargs)
    if not isinstance(outputs, (tuple, list)):
        outputs = (outputs,)
    torch.cuda.synchronize()
    return [o.detach().cpu().numpy() for o in outputs]

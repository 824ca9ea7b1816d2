"""Carrier types for models whose outputs are not plain tensors.

Same surface as tspipe/model_wrapper.py:7-27: a wrapped model may return any
nested structure; it travels through the pipeline as a ``TSPipeModelOutput``
whose ``lst_require_grad_tensor_path`` names the tensors that need gradients
(filled in later by the pipeline, tspipe/gpu_task.py:131-143).
"""
from dataclasses import dataclass
from typing import Any, List, Optional, Tuple, Union

import torch
from torch import nn


@dataclass
class TSPipeModelOutput:
    data: Any
    lst_require_grad_tensor_path: Optional[List[Tuple]]


class TSPipeModelWrapper(nn.Module):
    """Feeds ``input.data`` to the model when handed a ``TSPipeModelOutput`` and
    wraps every non-tensor result into one (tensors pass through bare)."""

    def __init__(self, model: nn.Module):
        super().__init__()
        self.model = model

    def forward(self, input) -> Union[TSPipeModelOutput, torch.Tensor]:
        payload = input.data if isinstance(input, TSPipeModelOutput) else input
        result = self.model.forward(payload)
        if isinstance(result, torch.Tensor):
            return result
        return TSPipeModelOutput(data=result, lst_require_grad_tensor_path=None)

"""Carrier types for models whose outputs are not plain tensors.

A wrapped model may return any nested structure (DistilBERT returns a dict of
logits and hidden states); it travels through the pipeline as a
``TSPipeModelOutput`` whose ``lst_require_grad_tensor_path`` names the tensors
that need gradients.  The pipeline fills that list in later
(tspipe/gpu_task.py:131-143); the wrapper always starts it as ``None``.
Field names, equality and ``repr`` follow tspipe/model_wrapper.py:7-10, because
the objects are pickled between TSPipe's worker processes.
"""
import dataclasses
from typing import Any, Callable, List, Optional, Tuple, Union

from torch import Tensor, nn

TensorPath = Tuple[Any, ...]


@dataclasses.dataclass
class TSPipeModelOutput:
    data: Any
    lst_require_grad_tensor_path: Optional[List[TensorPath]]

    def with_data(self, data: Any) -> "TSPipeModelOutput":
        """The same carrier (same gradient paths) around other content."""
        return dataclasses.replace(self, data=data)

    @staticmethod
    def unwrap(value: Any) -> Any:
        """``value.data`` for a carrier, ``value`` itself for anything else."""
        return value.data if isinstance(value, TSPipeModelOutput) else value


class TSPipeModelWrapper(nn.Module):
    """Adapter between a model with structured outputs and the pipeline
    (tspipe/model_wrapper.py:13-27): a carrier handed in is opened before the
    model sees it, tensors come back bare, and every other result leaves as a
    fresh carrier without gradient paths."""

    def __init__(self, model: nn.Module):
        super().__init__()
        self.model = model

    def forward(self, input) -> Union[TSPipeModelOutput, Tensor]:
        # the reference calls .forward directly, i.e. without the wrapped module's hooks
        run: Callable[[Any], Any] = self.model.forward
        result = run(TSPipeModelOutput.unwrap(input))
        if isinstance(result, Tensor):
            return result
        return TSPipeModelOutput(result, None)

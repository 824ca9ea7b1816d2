"""The names tspipe/model_wrapper.py exports, for ``from ...model_wrapper import``."""
from ._outputs import TSPipeModelOutput, TSPipeModelWrapper

__all__ = ["TSPipeModelOutput", "TSPipeModelWrapper"]

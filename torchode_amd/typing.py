"""Names for the tensors that travel through a solve, for annotations in user code.

The reference spells out shapes and dtypes with an annotation library (torchode/typing.py:44-95); here each
name is plain ``torch.Tensor`` and the shape is said in this table, so that ``from torchode_amd.typing import *``
keeps a user's plug-in importable:

    DataTensor             [batch, feature]         float
    NormTensor             [batch]                  float
    SolutionDataTensor     [batch, time, feature]   float
    TimeTensor             [batch]                  float
    EvaluationTimesTensor  [batch, time]            float
    AcceptTensor           [batch]                  bool
    StatusTensor           [batch]                  int64
    InterpTimeTensor       [n]                      float   (one entry per evaluation point that a step passed)
    InterpDataTensor       [n, feature]             float
    SampleIndexTensor      [n]                      int64   (which sample each of those points belongs to)
"""
from typing import Callable, Optional

import torch

DataTensor = NormTensor = SolutionDataTensor = TimeTensor = EvaluationTimesTensor = torch.Tensor
AcceptTensor = StatusTensor = InterpTimeTensor = InterpDataTensor = SampleIndexTensor = torch.Tensor


def _all_neighbours(tensors, same: Callable) -> bool:
    return all(same(a, b) for a, b in zip(tensors, tensors[1:]))


def same_dtype(*tensors: torch.Tensor) -> bool:
    return _all_neighbours(tensors, lambda a, b: a.dtype == b.dtype)


def same_device(*tensors: torch.Tensor) -> bool:
    return _all_neighbours(tensors, lambda a, b: a.device == b.device)


def same_shape(*tensors: torch.Tensor, dim: Optional[int] = None) -> bool:
    """Equal shapes, or equal sizes along ``dim`` only (reference typing.py:25-36)."""
    if dim is None:
        return _all_neighbours(tensors, lambda a, b: a.shape == b.shape)
    return _all_neighbours(tensors, lambda a, b: a.shape[dim] == b.shape[dim])

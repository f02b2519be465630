"""MI355X-native implementation of PiPPy's per-stage pipeline hot path.

Public names mirror ``pippy/__init__.py:2-43`` of the reference so that a script written against
``pippy`` runs against this package by changing the import.  All stages of a pipeline run as
virtual stages on one GPU; see ``schedules.py``.
"""
from . import _debug  # noqa: F401  (sets the logging level from PIPPY_VERBOSITY)
from ._IR import (ArgsChunkSpec, KwargsChunkSpec, Pipe, PipeSplitWrapper, SplitPoint,
                  annotate_split_points, pipe_split, pipeline)
from ._split_policies import split_by_graph, split_into_equal_size, split_on_size_threshold
from .losses import CrossEntropyLoss
from .optim import FusedAdamW, FusedSGD
from .microbatch import TensorChunkSpec, merge_chunks, split_args_kwargs_into_chunks, sum_reducer
from .schedules import (Schedule1F1B, ScheduleGPipe, ScheduleInterleaved1F1B, ScheduleLoopedBFS,
                        ScheduleZeroBubble)
from .stage import ManualPipelineStage, PipelineStage, VirtualGroup

__version__ = "0.1.0"

__all__ = [
    "Pipe", "pipe_split", "SplitPoint", "annotate_split_points", "pipeline", "ArgsChunkSpec",
    "KwargsChunkSpec", "TensorChunkSpec", "PipelineStage", "ManualPipelineStage", "Schedule1F1B",
    "ScheduleGPipe", "ScheduleInterleaved1F1B", "ScheduleLoopedBFS", "ScheduleZeroBubble",
    "split_args_kwargs_into_chunks", "merge_chunks", "sum_reducer", "CrossEntropyLoss",
    "VirtualGroup", "PipeSplitWrapper", "FusedSGD", "FusedAdamW", "split_into_equal_size",
    "split_on_size_threshold", "split_by_graph",
]

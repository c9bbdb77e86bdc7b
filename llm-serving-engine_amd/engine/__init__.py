from .batch import CacheCell, GroupBatch, SequenceChunk, StepBatch
from .runner import ModelRunner, StepEntry, build_step_batch

__all__ = ["CacheCell", "GroupBatch", "ModelRunner", "SequenceChunk", "StepBatch", "StepEntry", "build_step_batch"]

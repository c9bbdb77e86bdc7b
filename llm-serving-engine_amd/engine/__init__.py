from .batch import CacheCell, GroupBatch, SequenceChunk, StepBatch
from .llm_engine import EngineCore, LLMEngine, TokenEvent
from .runner import ModelRunner, StepEntry, build_step_batch
from .scheduler import IterationScheduler, RequestState, choose_victim, plan_iteration
from .tokenizer import ByteTokenizer, FileTokenizer, Tokenizer

__all__ = [
    "ByteTokenizer",
    "CacheCell",
    "EngineCore",
    "FileTokenizer",
    "GroupBatch",
    "IterationScheduler",
    "LLMEngine",
    "ModelRunner",
    "RequestState",
    "SequenceChunk",
    "StepBatch",
    "StepEntry",
    "TokenEvent",
    "Tokenizer",
    "build_step_batch",
    "choose_victim",
    "plan_iteration",
]

from .batch import CacheCell, GroupBatch, SequenceChunk, StepBatch
from .llm_engine import EngineCore, LLMEngine, RequestTooLongError, TokenEvent
from .runner import ModelRunner, StepEntry, build_step_batch
from .scheduler import Request, Scheduler, Share
from .tokenizer import ByteTokenizer, FileTokenizer, Tokenizer

__all__ = [
    "ByteTokenizer",
    "CacheCell",
    "EngineCore",
    "FileTokenizer",
    "GroupBatch",
    "LLMEngine",
    "ModelRunner",
    "Request",
    "RequestTooLongError",
    "Scheduler",
    "SequenceChunk",
    "Share",
    "StepBatch",
    "StepEntry",
    "TokenEvent",
    "Tokenizer",
    "build_step_batch",
]

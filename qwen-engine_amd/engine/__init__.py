from .batch import SeqInfo, StepContext
from .runner import ModelRunner, StepEntry, load_model, torch_dtype
from .scheduler import Planned, Request, Scheduler
from .llm_engine import GenerationResult, LLMEngine, generate, load_tokenizer

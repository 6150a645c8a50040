from .batch import SeqInfo, StepContext
from .runner import ModelRunner, StepEntry, load_model, torch_dtype

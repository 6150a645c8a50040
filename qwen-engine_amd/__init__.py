"""An inference engine for the Qwen3 dense decoder on one AMD MI355X (gfx950):
typed configuration and architecture registry, weights by tensor name, layers put
together from parts, a paged cache manager, one step function, a scheduler with
sampling, and trace replay; all device work in hand-written HIP kernels."""
from . import config, cache
from .config import EngineConfig, Qwen3Config, config_from_folder, register_architecture
from .sampling import SamplingParams
from .engine import GenerationResult, LLMEngine, ModelRunner, StepEntry, generate, load_model

__version__ = "0.1.0"

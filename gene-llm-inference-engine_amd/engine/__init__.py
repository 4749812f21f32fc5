"""Model assembly, the step function, the scheduler and the single-request loop."""
from .model import DecoderModel, compute_dtype, load_model, random_model
from .runner import Runner, StepEntry, StepError
from .generate import GenerateResult, generate
from .scheduler import POOL_TOO_SMALL, Engine, EngineConfig, EngineRequest, EngineResult, EngineStats

from .generator import Generator, SequenceState, plan_batches, plan_prompt_steps  # noqa: F401
from .model import DecoderModel, declared_weights  # noqa: F401
from .step import Engine, StepEntry  # noqa: F401

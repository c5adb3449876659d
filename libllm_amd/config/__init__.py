from .llama import LlamaConfig
from .registry import (architectures, config_from_dict, config_from_dir,  # noqa: F401
                       register_architecture)
from .spec import (EmbeddingSpec, HeadSpec, LayerSpec, ModelSpec, PartSpec,  # noqa: F401
                   ScheduleEntry, default_schedule, validate_schedule)

register_architecture("llama", LlamaConfig)

from .engine_config import (ADMISSION_MARGIN_BLOCKS, BLOCK_SIZE, NUM_GPU_BLOCKS, EngineConfig)
from .model_config import (ConfigError, FeedForwardSpec, LayerSpec, MixerSpec, ModelPlan, NormSpec,
                           PartSpec, PositionSpec, ScheduleEntry)
from .registry import (known_architectures, plan_of, read_config, read_config_dict,
                       register_architecture)

from .model import ConfigError, Qwen2Config, read_key
from .layered import (BiasedAttentionConfig, DenseMlpConfig, LatentAttentionConfig, LayerConfig,
                      TopelornConfig, WindowConfig)
from .vekanex import VekanexConfig, VekanexLayer
from .futezen import FutezenConfig, FutezenLayer
from .vunadra import VunadraConfig, VunadraLayer
from .engine import CacheConfig, SchedulerConfig, EngineConfig, PAGE_SIZES
from .registry import (Architecture, register_architecture, registered_architectures,
                       resolve_architecture)

# reference name for the model configuration (servelab/config.py:10)
ModelConfig = Qwen2Config

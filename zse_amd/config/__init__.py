from .base import (ARCHITECTURES, Architecture, ConfigError, load_config, read_config_json,
                   register_architecture, resolve_architecture, unregister_architecture)
from .plan import (AttentionSpec, BlockSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerCall,
                   ModelPlan, NoPositionSpec, NormSpec, RotarySpec)

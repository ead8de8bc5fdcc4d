from .lfm2 import Lfm2Config, adjusted_ff_dim
from .registry import (architecture_of, load_config, register_architecture, registered_architectures,
                       unregister_architecture)
from .spec import (AttentionSpec, BlockSpec, LayerCall, ModelSpec, NoPositionSpec, RMSNormSpec, RopeSpec,
                   ShortConvSpec, SwiGLUSpec)

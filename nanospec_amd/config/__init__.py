from .registry import architectures, load_config, register_architecture, resolve
from .llama import LlamaConfig  # (importing an architecture's module registers it)
from .vuzelix import VuzelixConfig
from .fetitar import FetitarConfig
from .padetar import PadetarConfig
from .fimilorn import FimilornConfig
from .spec import (AttentionSpec, ChannelDeltaSpec, DenseFFSpec, LatentAttentionSpec, LayerCall, ModelSpec, NoPositionSpec, PreNormBlockSpec, RMSNormSpec,
                   RopeSpec, StreamBlockSpec, SwiGLUSpec)

__all__ = [
    "LlamaConfig", "VuzelixConfig", "FetitarConfig", "PadetarConfig", "FimilornConfig", "LatentAttentionSpec", "ChannelDeltaSpec", "DenseFFSpec", "StreamBlockSpec", "architectures", "load_config", "register_architecture", "resolve", "AttentionSpec", "LayerCall",
    "ModelSpec", "NoPositionSpec", "PreNormBlockSpec", "RMSNormSpec", "RopeSpec", "SwiGLUSpec",
]

from .fazezen import (ChunkedAttentionConfig, DenseConfig, FazezenConfig, FazezenLayer, LightningConfig, ParallelConfig,
                      RetentionConfig, Rotation, Stretch)
from .lfm2 import Lfm2Config, adjusted_ff_dim
from .makuzen import LatentAttentionConfig, MakuzenConfig, MakuzenLayer, TableMoEConfig, YarnScaling
from .registry import (architecture_of, load_config, register_architecture, registered_architectures,
                       unregister_architecture)
from .spec import (AttentionSpec, BlockSpec, GatedMLPSpec, LatentAttentionSpec, LayerCall, LinearAttentionSpec, MixerPairSpec,
                   ModelSpec, NoPositionSpec, OutNormBlockSpec, ParallelBlockSpec, RMSNormSpec, RopeSpec, ScaledRopeSpec,
                   ShortConvSpec, StretchedRopeSpec, SwiGLUSpec, TableMoESpec)

from .fazezen import (ChunkedAttentionConfig, DenseConfig, FazezenConfig, FazezenLayer, LightningConfig, ParallelConfig,
                      RetentionConfig, Rotation, Stretch)
from .kuditar import (ChannelDecayConfig, DeltaRuleConfig, DenseFFConfig, GatedAttentionConfig, KuditarConfig, KuditarLayer,
                      PairConfig, RunAttentionConfig, SigmoidMoEConfig, Turn, WindowedAttentionConfig)
from .lfm2 import Lfm2Config, adjusted_ff_dim
from .makuzen import LatentAttentionConfig, MakuzenConfig, MakuzenLayer, TableMoEConfig, YarnScaling
from .registry import (architecture_of, load_config, register_architecture, registered_architectures,
                       unregister_architecture)
from .togalorn import ExpertConfig, LatentMixerConfig, LoopConfig, Mamba2MixerConfig, MoEConfig, TogalornConfig, TogalornLayer
from .spec import (AttentionSpec, BlockSpec, ClampedGLUSpec, GatedDeltaSpec, GatedLinearSpec, GatedMLPSpec, GroupRMSNormSpec,
                   LatentAttentionSpec, LayerCall, LayerNormSpec, LinearAttentionSpec, MixerPairSpec,
                   ModelSpec, NoPositionSpec, OutNormBlockSpec, ParallelBlockSpec, RMSNormSpec, ReentrySpec, RopeSpec,
                   RoutedMoESpec, ScaledRopeSpec, SharedNormBlockSpec, ShortConvSpec, StateSpaceSpec, StretchedRopeSpec,
                   SwiGLUSpec, TableMoESpec)

"""Typed configurations, the architecture registry and the neutral model description."""
from .spec import (AttentionSpec, DenseMlpSpec, GatedDeltaSpec, InterleavedRotarySpec, LatentAttentionSpec, LayerSpec, MlstmSpec, ModelSpec,
                   PartialRotarySpec, RejoinSpec, RmsNormSpec, RotarySpec, RoutedExpertsSpec, RunEntry, ScaleSpec, SelectiveScanSpec, SideBySideSpec, SoftCapSpec,
                   StreamAccessSpec, SwiGluSpec, TokenShiftSpec, TokenSideInputSpec)
from .errors import ConfigError
from .registry import (config_class_for, parse_config, read_config, register_architecture,
                       registered_architectures)
from .llama import Llama3Scaling, LlamaConfig          # registers itself
from .fekorax import FekoraxConfig                     # registers itself
from .rigalorn import RigalornConfig                   # registers itself
from .zidevik import ZidevikConfig                     # registers itself
from .mimitar import MimitarConfig                     # registers itself

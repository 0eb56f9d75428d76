"""Typed configurations and the architecture registry."""

from .plan import (  # noqa: F401
    AttentionSpec,
    CausalConvSpec,
    GateSpec,
    LatentAttentionSpec,
    RoutedFFNSpec,
    DenseFFNSpec,
    HeadSpec,
    LayerSpec,
    ModelPlan,
    NormSpec,
    OrderEntry,
    PositionSpec,
    TensorSource,
    TokenEmbeddingSpec,
)
from .registry import (  # noqa: F401
    architecture_name_of,
    config_from_dict,
    find_architecture,
    load_config,
    register_architecture,
    supported_architectures,
)
from .gpt2 import GPT2Config  # noqa: F401  (registers itself)
from .bokulix import BokulixConfig  # noqa: F401  (registers itself)
from .mofulix import MofulixConfig  # noqa: F401  (registers itself)
from .dopilorn import DopilornConfig  # noqa: F401  (registers itself)
from .larulorn import LarulornConfig  # noqa: F401  (registers itself)

"""Model parts: mixers, feed-forwards, norms, position encodings, blocks."""

from .base import GroupStep, PartStepPlan, StepContext, StepFacts, StepHost, Workspace  # noqa: F401
from .registry import (  # noqa: F401
    build_part,
    find_part,
    register_block,
    register_conv,
    register_embedding,
    register_entry,
    register_ffn,
    register_gate,
    register_head,
    register_mixer,
    register_norm,
    register_position,
)
from .norms import Normed, as_tensor  # noqa: F401
from . import (attention, block, conv, delta_rule, differential_attention, embeddings, feedforward, gated_recurrence, head, latent_attention, norms, recurrent, reentry,  # noqa: F401
               routed, scored_attention, side_by_side)  # noqa: F401  (register themselves)

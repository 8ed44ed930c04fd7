"""MI355X-native hot path of Recurrent Drafting behind the reference's Python call surface.

    import recurrent_drafting_amd as recurrent_drafting

Modules carry the reference's names: attention, configuration_drafter, kv_cache, modeling_drafter,
modeling_llama, recurrent_drafting, rng, stats, tree_attention.  The numerical work of the decode
step is done by libredrafter_hip.so (hand-written HIP kernels for gfx950); there is no CPU path.
"""

from . import (  # noqa: F401
    _hip,
    acceptance,
    attention,
    configuration_drafter,
    gemm_tuning,
    kv_cache,
    modeling_drafter,
    modeling_llama,
    packed_rows,
    recurrent_drafting,
    rng,
    stats,
    tree_attention,
)
from .modeling_drafter import BeamShape  # noqa: F401
from .recurrent_drafting import RecurrentDrafting, SamplingArgs, SpecialTokens  # noqa: F401

"""MI355X-native hot path of Recurrent Drafting behind the reference's Python call surface.

    import recurrent_drafting_amd as recurrent_drafting

Modules carry the reference's names: attention, kv_cache, modeling_drafter, modeling_llama,
recurrent_drafting, tree_attention.  The numerical work is done by libredrafter_hip.so.
"""

from . import _hip, tree_attention  # noqa: F401

__all__ = ["tree_attention"]

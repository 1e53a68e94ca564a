"""Drop-in for the reference package ``flash_recontruction`` (sic): same twelve exported names
(reference flash_recontruction/__init__.py:1-34) plus ``gqa_xKV_rope`` for the fused RoPE decode.
The v1..v4 aliases all bind to the one HIP implementation of each function."""
from .qAB_no_pe.v1 import qAB as qAB_no_pe_v1
from .qAB_no_pe.v2 import qAB_v3 as qAB_no_pe_v2
from .qAB_no_pe.ref import qAB_ref as qAB_no_pe_ref
from .qAB.v1 import qAB as qAB_rope_v1
from .qAB.v2 import qAB_precomp as qAB_rope_v2
from .qAB.v3 import qAB as qAB_rope_v3
from .qAB.v4 import qAB as qAB_rope_v4
from .fused_attention.no_pe.ref import group_query_attention_xKV as gqa_xKV_no_pe_ref
from .fused_attention.no_pe.ref import group_query_attention_xKV_k_only as gqa_xKV_no_pe_k_only_ref
from .fused_attention.no_pe.v1_k_only import decode_attention_fwd as gqa_xKV_no_pe_k_only
from .fused_attention.no_pe.v1 import decode_attention_fwd as gqa_xKV_no_pe
from .fused_attention.no_pe.v2 import decode_attention_fwd as gqa_xKV_no_pe_v2
from .fused_attention.rope.v1 import decode_attention_fwd as gqa_xKV_rope

__all__ = [
    "qAB_no_pe_v1", "qAB_no_pe_v2", "qAB_no_pe_ref",
    "qAB_rope_v1", "qAB_rope_v2", "qAB_rope_v3", "qAB_rope_v4",
    "gqa_xKV_no_pe_ref", "gqa_xKV_no_pe_k_only_ref", "gqa_xKV_no_pe_k_only",
    "gqa_xKV_no_pe", "gqa_xKV_no_pe_v2", "gqa_xKV_rope",
]

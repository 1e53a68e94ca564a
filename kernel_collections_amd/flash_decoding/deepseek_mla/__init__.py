"""Split-K decode with a separate buffer for recently decoded tokens (reference flash_decoding/deepseek_mla/).
The reference leaves this ``__init__`` empty; the entry points live in ``flash_decoding.py``."""
from .flash_decoding import (mla_decode_attention_fwd, mla_decode_attention_fwd_pd_sep,  # noqa: F401
                             mla_decode_attention_fwd_pd_sep_xKV)

from .mla_flash_decoding import mla_decode_attention_fwd, mla_decode_attention_xKV  # noqa: F401
from .stage1 import decoding_stage1  # noqa: F401
from .stage2 import decoding_stage2  # noqa: F401
from .ref import mla_decode_attention_fwd_ref  # noqa: F401

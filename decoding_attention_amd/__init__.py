"""MI355X-native single-query (decoding) attention: MHA / GQA / MQA / MLA over packed variable-length KV."""
__version__ = "0.1.0"

from .interface import (decoding_attn_fwd, decoding_attn_paged_fwd, fwd, pack_int4,  # noqa: F401
                        quantize_int4_per_group, quantize_int4_per_token, quantize_int8_per_group,
                        quantize_int8_per_token)

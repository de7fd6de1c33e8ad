"""Drop-in import name of the reference package: `from decoding_attn import decoding_attn_fwd`
(reference decoding_attn/__init__.py:15-19), served by the gfx950 library."""
__version__ = "0.1.0"

from decoding_attention_amd.interface import decoding_attn_fwd  # noqa: F401

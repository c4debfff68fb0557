# Same two names the reference package exports
# (custom_models/sba/stickbreaking_attention/__init__.py:1-2).
from .sb_attn import sb_attn, sb_attn_  # noqa: F401
from .sb_varlen import sb_attn_varlen, sb_attn_varlen_  # noqa: F401

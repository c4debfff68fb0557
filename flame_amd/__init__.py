"""MI355X-native stick-breaking attention: drop-in for the operator that
custom_models/sba of fla-org/flame calls (sb_attn / sb_attn_varlen)."""
from .stickbreaking_attention import sb_attn, sb_attn_varlen  # noqa: F401

__all__ = ["sb_attn", "sb_attn_varlen"]

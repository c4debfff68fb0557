"""``SBAConfig``: the fields and defaults of custom_models/sba/config_sba.py:7-69, so that the
reference's configs/sba_340m.json loads unchanged.  The three ``fuse_*`` switches are accepted
and kept (they select fla's fused kernels in the reference); here the plain PyTorch forms
are always used."""
from typing import Optional

from transformers.configuration_utils import PretrainedConfig


class SBAConfig(PretrainedConfig):
    model_type = 'sba'
    keys_to_ignore_at_inference = ['past_key_values']

    def __init__(self, hidden_size: int = 2048, num_hidden_layers: int = 24, num_heads: int = 32,
                 num_kv_heads: Optional[int] = None, qkv_bias: bool = False, window_size: Optional[int] = None,
                 rope_theta: Optional[float] = 10000., max_position_embeddings: int = 2048,
                 hidden_ratio: Optional[int] = 4, intermediate_size: Optional[int] = None,
                 hidden_act: str = "swish", initializer_range: float = 0.006,
                 elementwise_affine: Optional[bool] = True, norm_eps: float = 1e-6, use_cache: bool = True,
                 pad_token_id: Optional[int] = None, bos_token_id: int = 1, eos_token_id: int = 2,
                 tie_word_embeddings: bool = False, fuse_norm: bool = True, fuse_swiglu: bool = True,
                 fuse_cross_entropy: bool = True, vocab_size: int = 32000, **kwargs):
        self.hidden_size, self.num_hidden_layers, self.num_heads = hidden_size, num_hidden_layers, num_heads
        self.num_kv_heads, self.qkv_bias, self.window_size = num_kv_heads, qkv_bias, window_size
        self.rope_theta, self.max_position_embeddings = rope_theta, max_position_embeddings
        self.hidden_ratio, self.intermediate_size, self.hidden_act = hidden_ratio, intermediate_size, hidden_act
        self.initializer_range, self.elementwise_affine, self.norm_eps = initializer_range, elementwise_affine, norm_eps
        self.use_cache = use_cache
        self.fuse_norm, self.fuse_swiglu, self.fuse_cross_entropy = fuse_norm, fuse_swiglu, fuse_cross_entropy
        self.vocab_size = vocab_size
        super().__init__(pad_token_id=pad_token_id, bos_token_id=bos_token_id, eos_token_id=eos_token_id,
                         tie_word_embeddings=tie_word_embeddings, **kwargs)

    def mlp_width(self) -> int:
        """fla's GatedMLP rule: 2/3 * hidden_ratio * hidden, rounded up to a multiple of 256."""
        if self.intermediate_size is not None:
            return self.intermediate_size
        w = int(self.hidden_size * (self.hidden_ratio or 4) * 2 / 3)
        return 256 * ((w + 255) // 256)

"""``SBAModel`` / ``SBAForCausalLM`` as ``transformers.PreTrainedModel``s
(custom_models/sba/modeling_sba.py:96-407): the same blocks as flame_amd.modeling_sba (plain
PyTorch norm / SwiGLU / cross-entropy around the HIP stick-breaking attention), with the
Hugging Face config, weight initialisation, output classes and ``from_config`` / ``save_pretrained``
plumbing that flame's trainer relies on.  ``cu_seqlens`` (and ``max_seqlen``) pass through to the
attention layers, which the reference's layer refuses (sba_layer.py:86-87)."""
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F
from transformers.modeling_outputs import BaseModelOutputWithPast, CausalLMOutputWithPast
from transformers.modeling_utils import PreTrainedModel

from ..modeling_sba import SBABlock
from .configuration_sba import SBAConfig


class SBAPreTrainedModel(PreTrainedModel):
    config_class = SBAConfig
    base_model_prefix = 'model'
    supports_gradient_checkpointing = False
    _no_split_modules = ['SBABlock']

    def _init_weights(self, module):
        # modeling_sba.py:120-127: N(0, initializer_range) for Linear and Embedding weights
        if isinstance(module, nn.Linear):
            nn.init.normal_(module.weight, mean=0.0, std=self.config.initializer_range)
            if module.bias is not None:
                nn.init.zeros_(module.bias)
        elif isinstance(module, nn.Embedding):
            nn.init.normal_(module.weight, mean=0.0, std=self.config.initializer_range)


class SBAModel(SBAPreTrainedModel):
    def __init__(self, config: SBAConfig):
        super().__init__(config)
        self.embeddings = nn.Embedding(config.vocab_size, config.hidden_size, config.pad_token_id)
        self.layers = nn.ModuleList([SBABlock(config, i) for i in range(config.num_hidden_layers)])
        self.norm = nn.RMSNorm(config.hidden_size, eps=config.norm_eps)
        self.post_init()

    def get_input_embeddings(self):
        return self.embeddings

    def set_input_embeddings(self, value):
        self.embeddings = value

    def forward(self, input_ids: Optional[torch.LongTensor] = None, attention_mask: Optional[torch.Tensor] = None,
                inputs_embeds: Optional[torch.FloatTensor] = None, return_dict: Optional[bool] = None, **kwargs):
        if attention_mask is not None and not bool(attention_mask.all()):
            raise ValueError("SBA takes no padding mask; pack the batch and pass cu_seqlens")
        if (input_ids is None) == (inputs_embeds is None):
            raise ValueError("give exactly one of input_ids and inputs_embeds")
        x = self.embeddings(input_ids) if inputs_embeds is None else inputs_embeds
        layer_kwargs = {k: v for k, v in kwargs.items() if k in ('cu_seqlens', 'max_seqlen')}
        for layer in self.layers:
            x = layer(x, **layer_kwargs)
        x = self.norm(x)
        if return_dict is False:
            return (x,)
        return BaseModelOutputWithPast(last_hidden_state=x, past_key_values=None)


class SBAForCausalLM(SBAPreTrainedModel):
    # target -> source, the form transformers 5 expects (a bare list of names fails in its tie_weights())
    _tied_weights_keys = {'lm_head.weight': 'model.embeddings.weight'}

    def __init__(self, config: SBAConfig):
        super().__init__(config)
        self.model = SBAModel(config)
        self.vocab_size = config.vocab_size
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        self.post_init()

    def get_input_embeddings(self):
        return self.model.embeddings

    def set_input_embeddings(self, value):
        self.model.embeddings = value

    def get_output_embeddings(self):
        return self.lm_head

    def set_output_embeddings(self, new_embeddings):
        self.lm_head = new_embeddings

    def forward(self, input_ids: Optional[torch.LongTensor] = None, attention_mask: Optional[torch.Tensor] = None,
                inputs_embeds: Optional[torch.FloatTensor] = None, labels: Optional[torch.LongTensor] = None,
                return_dict: Optional[bool] = None, **kwargs):
        hidden = self.model(input_ids=input_ids, attention_mask=attention_mask, inputs_embeds=inputs_embeds,
                            return_dict=True, **kwargs).last_hidden_state
        logits = self.lm_head(hidden)
        loss = None
        if labels is not None:
            # modeling_sba.py:391: labels shifted left by one, the last position ignored
            shifted = torch.cat((labels[..., 1:], torch.full_like(labels[:, :1], -100)), 1)
            loss = F.cross_entropy(logits.view(shifted.numel(), -1).float(), shifted.view(-1), ignore_index=-100)
        if return_dict is False:
            return (loss, logits) if loss is not None else (logits,)
        return CausalLMOutputWithPast(loss=loss, logits=logits, past_key_values=None)

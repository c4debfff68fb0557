"""Hugging Face registration of the SBA model, as custom_models/sba/__init__.py:1-9 does it:
importing this package makes ``AutoConfig`` / ``AutoModel`` / ``AutoModelForCausalLM`` know
``model_type = 'sba'``, which is how flame's trainer finds a custom model
(flame/train.py:66-67, ``--experimental.custom_model_path``)."""
from transformers import AutoConfig, AutoModel, AutoModelForCausalLM

from .configuration_sba import SBAConfig
from .modeling_sba import SBAForCausalLM, SBAModel

__all__ = ['SBAConfig', 'SBAForCausalLM', 'SBAModel']

AutoConfig.register('sba', SBAConfig, exist_ok=True)
AutoModel.register(SBAConfig, SBAModel, exist_ok=True)
AutoModelForCausalLM.register(SBAConfig, SBAForCausalLM, exist_ok=True)

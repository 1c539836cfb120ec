from .llama.model import LLaMADecoderLayer, LLaMAForCausalLM, LLaMAModel
from .narurax.model import NaruraxConfig, NaruraxForCausalLM
from .quantized.quant import smooth_quantize, weight_only_quantize
from .registry import MODEL_REGISTRY, load_model, model_class_for
from .rofozen.model import RofozenConfig, RofozenForCausalLM
from .tolenex.model import TolenexConfig, TolenexForCausalLM
from .vetipel.model import VetipelConfig, VetipelForCausalLM

__all__ = ['LLaMADecoderLayer', 'LLaMAForCausalLM', 'LLaMAModel', 'smooth_quantize', 'weight_only_quantize', 'MODEL_REGISTRY',
           'load_model', 'model_class_for', 'TolenexConfig', 'TolenexForCausalLM',
           'VetipelConfig', 'VetipelForCausalLM', 'RofozenConfig', 'RofozenForCausalLM',
           'NaruraxConfig', 'NaruraxForCausalLM']

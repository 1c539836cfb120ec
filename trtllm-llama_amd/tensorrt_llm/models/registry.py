"""Which model class serves a checkpoint: looked up by what its config.json calls itself.

LLaMA checkpoints (HF layout: "architectures": ["LlamaForCausalLM"]) go through the builder of examples/llama_quant into a
GenerationSession; stack-engine designs (config key "architecture") are served by RaggedGenerationSession."""
import json
import os

from .llama.model import LLaMAForCausalLM
from .narurax.model import NaruraxForCausalLM
from .rofozen.model import RofozenForCausalLM
from .tolenex.model import TolenexForCausalLM
from .vetipel.model import VetipelForCausalLM

MODEL_REGISTRY = {
    'LlamaForCausalLM': LLaMAForCausalLM,
    'LLaMAForCausalLM': LLaMAForCausalLM,
    'Narurax': NaruraxForCausalLM,
    'Rofozen': RofozenForCausalLM,
    'Tolenex': TolenexForCausalLM,
    'Vetipel': VetipelForCausalLM,
}


def architecture_of(config: dict) -> str:
    if 'architecture' in config:
        return config['architecture']
    archs = config.get('architectures') or []
    if archs:
        return archs[0]
    raise KeyError('config.json names no architecture ("architecture" or "architectures")')


def model_class_for(config: dict):
    name = architecture_of(config)
    if name not in MODEL_REGISTRY:
        raise KeyError(f'architecture {name!r} is not registered (known: {sorted(MODEL_REGISTRY)})')
    return MODEL_REGISTRY[name]


def load_model(model_dir: str):
    """The model object for a checkpoint directory whose class builds from a checkpoint (stack-engine designs)."""
    with open(os.path.join(model_dir, 'config.json')) as f:
        cls = model_class_for(json.load(f))
    if not hasattr(cls, 'from_checkpoint'):
        raise NotImplementedError(f'{cls.__name__} is built through its example\'s build.py, not from a checkpoint directory')
    return cls.from_checkpoint(model_dir)

"""Model registry: config.json -> the host layer that serves it.  A layer-list design names itself in `architecture`; the llama
family keeps Hugging Face's `architectures` list (the reference picks its model struct the same way,
src/openai/pipelines/pipeline.rs `DefaultLoader::load_model`)."""
import json
import os

_REGISTRY = {}
_COMPONENT = {}


def register(name, loader, component=None):
    """loader(model_dir, config, **options) -> model; component: the part of the library that serves the model when it can be built
    alone (`__graft_entry__.COMPONENTS`), None = the whole library"""
    _REGISTRY[name] = loader
    _COMPONENT[name] = component


def component_of(config):
    """which part of the library a config needs (None: the whole library, or nothing registered)"""
    for name in architectures_of(config):
        if name in _REGISTRY:
            return _COMPONENT[name]
    return None


def architectures_of(config):
    names = []
    if isinstance(config.get("architecture"), str):
        names.append(config["architecture"])
    names += [a for a in config.get("architectures", []) if isinstance(a, str)]
    return names


def registered():
    return sorted(_REGISTRY)


def load_model(model_dir, **options):
    config = json.load(open(os.path.join(model_dir, "config.json")))
    for name in architectures_of(config):
        if name in _REGISTRY:
            return _REGISTRY[name](model_dir, config, **options)
    raise ValueError(f"no host layer registered for {architectures_of(config) or 'a config without an architecture'}; "
                     f"registered: {registered()}")


def _load_layer_list(model_dir, config, dtype="bfloat16", block_size=None, state_slots=4, **_):
    from .hybrid_model import HybridModel, DEFAULT_BLOCK_SIZE
    return HybridModel.from_pretrained(model_dir, dtype=dtype, block_size=block_size or DEFAULT_BLOCK_SIZE, state_slots=state_slots)


def _load_dense_llama(model_dir, config, dtype="bfloat16", **options):
    from .dense_loader import load_dense_llama
    return load_dense_llama(model_dir, config, dtype=dtype, **options)


for _name in ("Sogodra", "Vivazen", "Kerolorn", "Sabolorn"):
    register(_name, _load_layer_list, component="hybrid")
for _name in ("LlamaForCausalLM", "MistralForCausalLM", "Qwen2ForCausalLM"):
    register(_name, _load_dense_llama)

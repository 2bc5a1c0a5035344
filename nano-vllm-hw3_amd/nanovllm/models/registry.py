"""Which model class serves a checkpoint: config.json names its architecture ("architectures": [...] in the Hugging
Face layout, or a plain "architecture"), and the entry of that name gives the module and class.  A class may define
``normalize_config(dict) -> dict`` to bring its own config.json layout to the fields the engine reads
(vocab_size, hidden_size, max_position_embeddings, torch_dtype) and the class attributes
``runs_portions`` (it is stepped with portions of sequences, mixed freely, and keeps its own cache and state) and
``default_block_size`` (tokens per cache block)."""
import importlib

_MODELS = {
    "Qwen3ForCausalLM": ("nanovllm.models.qwen3", "Qwen3ForCausalLM"),
    "Qwen2ForCausalLM": ("nanovllm.models.qwen3", "Qwen3ForCausalLM"),      # the same decoder with qkv biases
    "Pasizen": ("nanovllm.models.pasizen", "PasizenForCausalLM"),
    "Lipelix": ("nanovllm.models.lipelix", "LipelixForCausalLM"),
    "Galupel": ("nanovllm.models.galupel", "GalupelForCausalLM"),
    "Lilevik": ("nanovllm.models.lilevik", "LilevikForCausalLM"),
}
DEFAULT = "Qwen3ForCausalLM"


def register(name, module, cls):
    _MODELS[name] = (module, cls)


def architecture_of(config: dict) -> str:
    names = config.get("architectures") or ([config["architecture"]] if config.get("architecture") else [])
    for n in names:
        if n in _MODELS:
            return n
    if names:
        raise ValueError(f"no model class for architecture {names}; known: {sorted(_MODELS)}")
    return DEFAULT


def model_class(name: str):
    module, cls = _MODELS[name]
    return getattr(importlib.import_module(module), cls)

from .llama import LlamaForCausalLM

# architecture name (config.json) -> (module, class). Anything not listed
# runs on the flag-driven llama-lineage graph.
_MODEL_CLASSES = {
    "Vunitar": ("vunitar", "VunitarForCausalLM"),
    "Fusipel": ("fusipel", "FusipelForCausalLM"),
    "Livasun": ("livasun", "LivasunForCausalLM"),
    "Makezen": ("makezen", "MakezenForCausalLM"),
}


def model_class_for(architecture: str):
    ent = _MODEL_CLASSES.get(architecture)
    if ent is None:
        return LlamaForCausalLM
    import importlib

    return getattr(importlib.import_module(f"{__name__}.{ent[0]}"), ent[1])


__all__ = ["LlamaForCausalLM", "model_class_for"]

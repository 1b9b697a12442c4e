"""Model registry: config.json names the architecture, the registry names the class that serves it.

A model class takes the loaded config in its constructor and offers ``forward(input_ids, positions)`` over the step's
Context.  Optional hooks a class may define (the runner and the loader look for them):
  requires_cache / has_recurrent_state   the step always reads paged caches / sequences own a state slot
  supported_dtypes                       activation types it can be served in (default: bf16 only)
  adapt_config(config, shapes)           sizes that only the checkpoint's tensor shapes give
  weight_target(name)                    checkpoint tensor name -> (parameter name, shard id)
  synthetic_tensors(config, ...)         random weights in checkpoint naming
  gather_rows / compute_logits_rows      logits of selected rows of what forward returns
"""
from __future__ import annotations

import importlib

_REGISTRY = {
    "Qwen3ForCausalLM": ("qwen3", "Qwen3ForCausalLM"),
    "Qwen2ForCausalLM": ("qwen3", "Qwen3ForCausalLM"),        # the same wiring with attention_bias (models/qwen3.py)
    "Lamutar": ("lamutar", "LamutarForCausalLM"),
    "LamutarForCausalLM": ("lamutar", "LamutarForCausalLM"),
    "Dinatar": ("dinatar", "DinatarForCausalLM"),
    "DinatarForCausalLM": ("dinatar", "DinatarForCausalLM"),
    "Lakatar": ("lakatar", "LakatarForCausalLM"),
    "LakatarForCausalLM": ("lakatar", "LakatarForCausalLM"),
    "Sokipel": ("sokipel", "SokipelForCausalLM"),
    "SokipelForCausalLM": ("sokipel", "SokipelForCausalLM"),
}


def architecture_of(hf_config) -> str:
    """The architecture a config names: ``architecture`` (a string) or the first of ``architectures``; configs that name
    none are taken for the Qwen3 family, the only one that ever came without."""
    name = getattr(hf_config, "architecture", None)
    if not name:
        names = getattr(hf_config, "architectures", None) or ["Qwen3ForCausalLM"]
        name = names[0]
    return name


def register(architecture: str, module: str, cls: str) -> None:
    _REGISTRY[architecture] = (module, cls)


def get_model_class(hf_config):
    name = architecture_of(hf_config)
    if name not in _REGISTRY:
        raise ValueError(f"architecture {name!r} is not served; known: {sorted(_REGISTRY)}")
    module, cls = _REGISTRY[name]
    return getattr(importlib.import_module(f"{__name__}.{module}"), cls)

"""Model registry: the architecture name a checkpoint's config.json carries -> the class that builds it and the reader
of its configuration.  ``Config`` resolves the configuration through ``read_config``; ``ModelRunner`` builds the model
through ``model_class``."""

import importlib

# architecture name -> (module, class name); modules are imported on first use
_MODELS = {
    "Qwen2ForCausalLM": ("byox_vllm_amd.models.qwen3", "Qwen3ForCausalLM"),
    "Qwen3ForCausalLM": ("byox_vllm_amd.models.qwen3", "Qwen3ForCausalLM"),
    "Rurutar": ("byox_vllm_amd.models.rurutar", "RurutarForCausalLM"),
    "Nonetar": ("byox_vllm_amd.models.nonetar", "NonetarForCausalLM"),
    "Zamusun": ("byox_vllm_amd.models.zamusun", "ZamusunForCausalLM"),
    "Kikelorn": ("byox_vllm_amd.models.kikelorn", "KikelornForCausalLM"),
}
DEFAULT = "Qwen3ForCausalLM"


def register(name: str, module: str, cls: str) -> None:
    _MODELS[name] = (module, cls)


def architecture_of(cfg) -> str:
    """The registry key of a configuration object or of a raw config.json dict."""
    get = cfg.get if isinstance(cfg, dict) else (lambda k, d=None: getattr(cfg, k, d))
    name = get("architecture") or (get("architectures") or [DEFAULT])[0]
    return name if name in _MODELS else DEFAULT


def model_class(cfg):
    module, cls = _MODELS[architecture_of(cfg)]
    return getattr(importlib.import_module(module), cls)


def read_config(raw: dict, path: str | None):
    """A model class may read its own configuration (``config_from_json(raw, path)``); the others get the HF reader."""
    cls = model_class(raw)
    reader = getattr(cls, "config_from_json", None)
    return reader(raw, path) if reader is not None else None

"""Model classes by the architecture name a configuration gives (the role of the reference's ModelRegistry,
python/sglang/srt/models/registry.py, reduced to the families this package has).  HuggingFace configurations name
theirs under "architectures"; Seturax, Verozen, Gatarax and Fudonex configurations under "architecture"."""
import importlib

_ARCHITECTURES = {
    "LlamaForCausalLM": ("llama", "LlamaForCausalLM"),
    "DeepseekV2ForCausalLM": ("deepseek_v2", "DeepseekV2ForCausalLM"),
    "DeepseekV3ForCausalLM": ("deepseek_v2", "DeepseekV2ForCausalLM"),
    "Seturax": ("seturax", "SeturaxForCausalLM"),
    "Verozen": ("verozen", "VerozenForCausalLM"),
    "Gatarax": ("gatarax", "GataraxForCausalLM"),
    "Fudonex": ("fudonex", "FudonexForCausalLM"),
}


def supported_architectures():
    return sorted(_ARCHITECTURES)


def get_model_class(architecture: str):
    try:
        module, name = _ARCHITECTURES[architecture]
    except KeyError:
        raise ValueError(f"unknown architecture {architecture!r}; this package has {supported_architectures()}") from None
    return getattr(importlib.import_module(f"{__package__}.{module}"), name)

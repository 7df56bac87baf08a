"""Model registry: arch config -> model class. The runner builds whatever the
checkpoint's config names; a new family registers here."""
from __future__ import annotations


def _llama():
    from .llama import LlamaForCausalLM

    return LlamaForCausalLM


def _dulotar():
    from .hybrid import DulotarForCausalLM

    return DulotarForCausalLM


def _nugopel():
    from .nugopel import NugopelForCausalLM

    return NugopelForCausalLM


def _vekusun():
    from .vekusun import VekusunForCausalLM

    return VekusunForCausalLM


def _vigonex():
    from .vigonex import VigonexForCausalLM

    return VigonexForCausalLM


MODEL_REGISTRY = {
    "llama": _llama,
    "mixtral": _llama,
    "dulotar": _dulotar,
    "nugopel": _nugopel,
    "vekusun": _vekusun,
    "vigonex": _vigonex,
}


def model_class(architecture: str):
    try:
        return MODEL_REGISTRY[architecture]()
    except KeyError:
        raise ValueError(
            f"no model class registered for architecture {architecture!r}; "
            f"known: {sorted(MODEL_REGISTRY)}"
        ) from None


# HIP extensions (kubeai_amd.<name>) whose kernels a family's forward uses
MODEL_EXTENSIONS = {
    "llama": ("_C",),
    "mixtral": ("_C",),
    "dulotar": ("_C_seq",),
    "nugopel": ("_C_seq",),
    "vekusun": ("_C_seq",),
    "vigonex": ("_C_seq",),
}


def required_extensions(architecture: str) -> tuple:
    return MODEL_EXTENSIONS.get(architecture, ("_C",))

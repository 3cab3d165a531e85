"""Model registry: architecture name (ModelArchConfig.arch /
HybridArchConfig.arch) -> model class. The engine builds whatever the
resolved config names; a new family registers here."""

from __future__ import annotations


def model_class(arch: str):
    if arch == "llama":
        from .llama import LlamaForCausalLM

        return LlamaForCausalLM
    if arch == "mixtral":
        from .mixtral import MixtralForCausalLM

        return MixtralForCausalLM
    if arch == "zutalix":
        from .zutalix import ZutalixForCausalLM

        return ZutalixForCausalLM
    if arch == "medilix":
        from .medilix import MedilixForCausalLM

        return MedilixForCausalLM
    if arch == "mitunex":
        from .mitunex import MitunexForCausalLM

        return MitunexForCausalLM
    if arch == "pironex":
        from .pironex import PironexForCausalLM

        return PironexForCausalLM
    raise ValueError(f"no model registered for architecture {arch!r}")


ARCHITECTURES = ("llama", "mixtral", "zutalix", "medilix", "mitunex", "pironex")

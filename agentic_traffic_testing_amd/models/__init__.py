"""Model registry: a configuration's ``family`` names the class that runs it."""
from __future__ import annotations


def model_class(family: str):
    if family == "llama":
        from .llama import LlamaModel

        return LlamaModel
    if family == "ledazen":
        from .ledazen import LedazenModel

        return LedazenModel
    if family == "soselix":
        from .soselix import SoselixModel

        return SoselixModel
    if family == "semezen":
        from .semezen import SemezenModel

        return SemezenModel
    if family == "lovapel":
        from .lovapel import LovapelModel

        return LovapelModel
    raise ValueError(f"no model registered for family {family!r}")


FAMILIES = ("llama", "ledazen", "soselix", "semezen", "lovapel")

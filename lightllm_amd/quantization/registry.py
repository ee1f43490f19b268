"""Name -> quantization method lookup.

Same surface as LightLLM's registry (lightllm/common/quantization/registry.py:4-32): a class decorator
``QUANTMETHODS.register(names, platform)`` and ``QUANTMETHODS.get(name, platform)`` that returns a fresh
instance and raises ValueError with the reference's messages for an unknown name or platform.
Entries are keyed by the (name, platform) pair.
"""
from typing import Dict, Iterable, Tuple, Union

from .quantize_method import QuantizationMethod


class QuantMethodFactory:
    def __init__(self):
        self._classes: Dict[Tuple[str, str], type] = {}

    def register(self, names: Union[str, Iterable[str]], platform: str = "cuda"):
        aliases = (names,) if isinstance(names, str) else tuple(names)

        def bind(cls):
            self._classes.update({(alias, platform): cls for alias in aliases})
            return cls

        return bind

    def names(self, platform: str = "cuda"):
        return sorted(name for name, plat in self._classes if plat == platform)

    def get(self, key, platform="cuda", *args, **kwargs) -> "QuantizationMethod":
        cls = self._classes.get((key, platform))
        if cls is not None:
            return cls()
        if any(name == key for name, _ in self._classes):
            raise ValueError(f"QuantMethod '{key}' for platform '{platform}' not supported.")
        raise ValueError(f"QuantMethod '{key}' not supported.")


QUANTMETHODS = QuantMethodFactory()

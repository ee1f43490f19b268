"""Name -> class registry of quantization methods (lightllm/common/quantization/registry.py:4-32)."""
from .quantize_method import QuantizationMethod


class QuantMethodFactory:
    def __init__(self):
        self._quant_methods = {}

    def register(self, names, platform="cuda"):
        def decorator(cls):
            for n in [names] if isinstance(names, str) else names:
                self._quant_methods.setdefault(n, {})[platform] = cls
            return cls

        return decorator

    def get(self, key, platform="cuda", *args, **kwargs) -> "QuantizationMethod":
        by_platform = self._quant_methods.get(key)
        if not by_platform:
            raise ValueError(f"QuantMethod '{key}' not supported.")
        cls = by_platform.get(platform)
        if cls is None:
            raise ValueError(f"QuantMethod '{key}' for platform '{platform}' not supported.")
        return cls()


QUANTMETHODS = QuantMethodFactory()

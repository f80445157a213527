"""Model registry: configuration family -> model class (the runner builds `model_class(cfg)`)."""


def model_class(cfg):
    family = getattr(cfg, "family", "llama")
    if family in ("llama", "mixtral"):
        from .llama import LlamaModel
        return LlamaModel
    if family == "vivepel":
        from .vivepel import VivepelModel
        return VivepelModel
    if family == "kafilorn":
        from .kafilorn import KafilornModel
        return KafilornModel
    if family == "suvapel":
        from .suvapel import SuvapelModel
        return SuvapelModel
    raise ValueError(f"no model class for family {family!r}")

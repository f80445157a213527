"""Model registry: configuration family -> model class (the runner builds `model_class(cfg)`)."""

# the families that keep their residual in fp32: they need only the small kernel library (build.build_mixers) and also
# run with DTYPE=float32; config.json's "architecture" of each
MIXER_FAMILIES = ("vivepel", "kafilorn", "suvapel", "zibinex")
MIXER_ARCHITECTURES = ("Vivepel", "Kafilorn", "Suvapel", "Zibinex")


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
    if family == "zibinex":
        from .zibinex import ZibinexModel
        return ZibinexModel
    raise ValueError(f"no model class for family {family!r}")

"""Model registry: configuration family -> model class."""


def model_class(family: str):
    if family == "mofidra":
        from .mofidra import MofidraModel
        return MofidraModel
    if family == "padadra":
        from .padadra import PadadraModel
        return PadadraModel
    if family == "mabivik":
        from .mabivik import MabivikModel
        return MabivikModel
    if family == "sitidra":
        from .sitidra import SitidraModel
        return SitidraModel
    from .transformer import DecoderModel
    return DecoderModel


def build_model(cfg, ops, device, dtype, tp=None, quant=None):
    """The model class that serves ``cfg`` (chosen by ``cfg.family``)."""
    return model_class(cfg.family)(cfg, ops, device, dtype, tp, quant=quant)

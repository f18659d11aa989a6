from dgi.models.config import (BebovikConfig, DepelixConfig, LofuvikConfig, ModelConfig, PRESETS,  # noqa: F401
                               TifepelConfig,
                               get_config)


def model_class(cfg):
    """The native model class that serves a configuration (the engine's model registry)."""
    if isinstance(cfg, BebovikConfig):
        from dgi.models.bebovik import BebovikModel
        return BebovikModel
    if isinstance(cfg, TifepelConfig):
        from dgi.models.tifepel import TifepelModel
        return TifepelModel
    if isinstance(cfg, DepelixConfig):
        from dgi.models.depelix import DepelixModel
        return DepelixModel
    if isinstance(cfg, LofuvikConfig):
        from dgi.models.lofuvik import LofuvikModel
        return LofuvikModel
    from dgi.models.llama import LlamaModel
    return LlamaModel


def build_model(cfg, device, dtype, layer_start: int = 0, layer_end=None, **kw):
    return model_class(cfg)(cfg, device, dtype, layer_start, layer_end, **kw)

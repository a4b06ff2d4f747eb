"""Native transformer, layer-list decoders, architecture configs and checkpoint interop."""
from .config import PRESETS, ModelConfig, preset  # noqa: F401
from .transformer import FlatParams, Transformer  # noqa: F401
from .hybrid import HybridConfig, HybridDecoder  # noqa: F401

# model family (``ModelConfig.family``) -> class; every family not listed is a ``Transformer`` variant
MODEL_CLASSES = {"kuzanex": HybridDecoder, "lufivik": HybridDecoder, "pobelorn": HybridDecoder,
                 "zusotar": HybridDecoder}


def model_class(cfg: ModelConfig):
    return MODEL_CLASSES.get(cfg.family, Transformer)


def build_model(cfg: ModelConfig, **kwargs):
    """The model object of a configuration's family."""
    return model_class(cfg)(cfg, **kwargs)

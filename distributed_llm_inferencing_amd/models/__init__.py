from .configs import ModelConfig, get_config, list_models  # noqa: F401
from .model import TransformerLM  # noqa: F401


def model_class(cfg):
    """The model class that runs ``cfg`` (the registry's arch -> implementation map)."""
    if cfg.is_hybrid:
        from .hybrid import HybridLM
        return HybridLM
    from .model import TransformerLM
    return TransformerLM

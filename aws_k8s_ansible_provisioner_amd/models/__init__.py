from .config import ModelConfig, get_config, list_models  # noqa: F401


def model_class(cfg: ModelConfig):
    """The model implementation that serves `cfg` (by its arch)."""
    if cfg.arch == "bidetar":
        from .bidetar import BidetarLM

        return BidetarLM
    if cfg.arch == "puputar":
        from .puputar import PuputarLM

        return PuputarLM
    if cfg.arch == "sazepel":
        from .sazepel import SazepelLM

        return SazepelLM
    if cfg.arch == "mudepel":
        from .mudepel import MudepelLM

        return MudepelLM
    from .transformer import DecoderLM

    return DecoderLM

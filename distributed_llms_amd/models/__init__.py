"""Model registry: the stage class that runs each architecture (``ModelConfig.arch``)."""


def stage_class(arch: str):
    if arch == "tudilix":
        from .hybrid import HybridStage
        return HybridStage
    if arch == "gikovik":
        from .gikovik import GikovikStage
        return GikovikStage
    if arch == "zebutar":
        from .zebutar import ZebutarStage
        return ZebutarStage
    if arch == "fekizen":
        from .fekizen import FekizenStage
        return FekizenStage
    if arch in ("llama", "mixtral", "gpt2"):
        from .stage import ModelStage
        return ModelStage
    raise KeyError(f"no stage class for architecture {arch!r}")


def make_stage(cfg, layer_start=0, layer_end=None, device="cpu", dtype=None, **kw):
    """The stage of ``cfg``'s architecture over layers [layer_start, layer_end) (None: to the last)."""
    import torch
    layer_end = cfg.num_layers if layer_end is None else layer_end
    return stage_class(cfg.arch)(cfg, layer_start, layer_end, device=device,
                                 dtype=torch.bfloat16 if dtype is None else dtype, **kw)

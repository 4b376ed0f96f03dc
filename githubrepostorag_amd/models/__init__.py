"""Model families served by the engine."""
from __future__ import annotations


def build_decoder(cfg, **kw):
    """Instantiate the decoder class for ``cfg.arch`` (same engine interface:
    forward / compute_logits / allocate_kv_cache / kv_bytes_per_block; models with recurrent state add
    allocate_state and ``has_state``)."""
    if cfg.arch == "gpt2":
        from .gpt2 import GPT2Model

        return GPT2Model(cfg, **kw)
    if cfg.arch == "zofesun":
        from .zofesun import ZofesunModel

        return ZofesunModel(cfg, **kw)
    if cfg.arch == "namudra":
        from .namudra import NamudraModel

        return NamudraModel(cfg, **kw)
    if cfg.arch == "leripel":
        from .leripel import LeripelModel

        return LeripelModel(cfg, **kw)
    if cfg.arch == "pubulix":
        from .pubulix import PubulixModel

        return PubulixModel(cfg, **kw)
    from .qwen2 import Qwen2Model

    return Qwen2Model(cfg, **kw)


def load_decoder(model_dir, device="cuda", dtype=None, **kw):
    """The decoder a checkpoint directory holds (config.json + safetensors): the class is chosen by the
    config, the weights are loaded with the safetensors reader (nothing in the file is executed)."""
    import torch

    from .configs import config_from_dir
    from .weights import load_state_dict

    cfg = config_from_dir(model_dir)
    sd = load_state_dict(model_dir, device=None)
    return build_decoder(cfg, device=device, dtype=dtype or torch.bfloat16, state_dict=sd, **kw)

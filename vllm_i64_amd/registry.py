"""Model registry: the architecture a checkpoint's config.json names -> the runner that serves it.

A loader takes (config dict, tensors by name, options) and returns a runner with the shared step interface
(`forward(token_ids, positions, slot_ids, ctx_len, logit_rows=..., tokens_per_seq=...)`, a paged cache `kv` with
reserve / free, `cfg.vocab_size`), which is all the engine, the decoders and the command line need."""
from __future__ import annotations

import json
import os
from typing import Callable, Dict, Optional

_LOADERS: Dict[str, Callable] = {}


def register(architecture: str, loader: Callable) -> None:
    _LOADERS[architecture.lower()] = loader


def architectures():
    return sorted(_LOADERS)


def architecture_of(config: dict) -> str:
    """The registry key of a config.json: 'architecture', else the first of 'architectures', else 'model_type'."""
    name = config.get("architecture") or (config.get("architectures") or [None])[0] or config.get("model_type")
    if not name:
        raise ValueError("config.json names no architecture ('architecture', 'architectures' or 'model_type')")
    return str(name)


def _load_morilorn(config: dict, tensors, *, device, dtype, max_seqs, max_tokens, kv_block=16, **_):
    from .config import MorilornConfig
    from .morilorn import MorilornModel
    cfg = MorilornConfig.from_dict(config)
    blocks = max(1, (int(max_tokens) + kv_block - 1) // kv_block)
    return MorilornModel(cfg, tensors, device=device, dtype=dtype, max_seqs=max_seqs, num_kv_blocks=blocks, kv_block=kv_block)


def _load_dogalorn(config: dict, tensors, *, device, dtype, max_seqs, max_tokens, kv_block=16, **_):
    from .config import DogalornConfig
    from .dogalorn import DogalornModel
    cfg = DogalornConfig.from_dict(config)
    blocks = max(1, (int(max_tokens) + kv_block - 1) // kv_block)
    return DogalornModel(cfg, tensors, device=device, dtype=dtype, max_seqs=max_seqs, num_kv_blocks=blocks, kv_block=kv_block)


def _load_zabutar(config: dict, tensors, *, device, dtype, max_seqs, max_tokens, kv_block=16, **_):
    from .config import ZabutarConfig
    from .zabutar import ZabutarModel
    config = dict(config)
    # sizes that the file may leave to the tensors' shapes
    for key, name, axis in (("vocab", "embed", 0), ("width", "embed", 1), ("max_positions", "pos", 0)):
        if key not in config and name in tensors:
            config[key] = int(tensors[name].shape[axis])
    if "canon" not in config and "l0.canon1" in tensors:
        config["canon"] = {"taps": int(tensors["l0.canon1"].shape[1])}
    cfg = ZabutarConfig.from_dict(config)
    blocks = max(1, (int(max_tokens) + kv_block - 1) // kv_block)
    return ZabutarModel(cfg, tensors, device=device, dtype=dtype, max_seqs=max_seqs, num_kv_blocks=blocks, kv_block=kv_block)


def _load_fukatar(config: dict, tensors, *, device, dtype, max_seqs, max_tokens, kv_block=16, **_):
    from .config import FukatarConfig
    from .fukatar import FukatarModel
    config = dict(config)
    for key, axis in (("vocab", 0), ("width", 1)):      # sizes that the file may leave to the tensors' shapes
        if key not in config and "embed" in tensors:
            config[key] = int(tensors["embed"].shape[axis])
    layers = []
    for i, l in enumerate(config.get("layers") or []):     # (the convolution's taps likewise, where a delta rule's entry leaves them out)
        name = f"l{i}.mix.right.q.conv"
        if l.get("type") == "parallel" and "conv" not in ((l.get("mixer") or {}).get("right") or {"conv": 0}) and name in tensors:
            l = dict(l, mixer=dict(l["mixer"], right=dict(l["mixer"]["right"], conv=int(tensors[name].shape[1]))))
        layers.append(l)
    config["layers"] = layers
    cfg = FukatarConfig.from_dict(config)
    blocks = max(1, (int(max_tokens) + kv_block - 1) // kv_block)
    return FukatarModel(cfg, tensors, device=device, dtype=dtype, max_seqs=max_seqs, num_kv_blocks=blocks, kv_block=kv_block)


def _load_complexity_deep(config: dict, tensors, *, device, dtype, max_seqs, max_tokens, quant="int8", **_):
    import torch
    from .checkpoint import config_from_dict, native_to_weights
    from .model import I64MoEModel
    cfg = config_from_dict(config)
    blocks = max(1, (int(max_tokens) + cfg.kv_block - 1) // cfg.kv_block)
    kv_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
    return I64MoEModel(cfg, native_to_weights(tensors, cfg), device=device, kv_dtype=kv_dtype, max_seqs=max_seqs, num_kv_blocks=blocks, quant=quant)


register("Morilorn", _load_morilorn)
register("Dogalorn", _load_dogalorn)
register("Zabutar", _load_zabutar)
register("Fukatar", _load_fukatar)
register("complexity-deep", _load_complexity_deep)
register("ComplexityDeepModel", _load_complexity_deep)


def load_model(path: str, *, dtype: str = "bfloat16", device="cuda:0", max_seqs: int = 4, max_tokens: int = 4096, config: Optional[dict] = None, **options):
    """The runner for the checkpoint folder `path` (config.json + tensors), chosen by its config.json."""
    from .checkpoint import read_state_dict
    if config is None:
        with open(os.path.join(path, "config.json"), "r", encoding="utf-8") as f:
            config = json.load(f)
    arch = architecture_of(config)
    loader = _LOADERS.get(arch.lower())
    if loader is None:
        raise ValueError(f"architecture '{arch}' is not registered (known: {architectures()})")
    return loader(config, read_state_dict(path), device=device, dtype=dtype, max_seqs=max_seqs, max_tokens=max_tokens, **options)

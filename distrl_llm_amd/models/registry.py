"""Model-class selection from a checkpoint directory's ``config.json``.

Dense Hugging Face families (``"architectures": ["Qwen2ForCausalLM"]`` ...)
load into :class:`CausalLM` and run on :class:`Engine`; layer-list designs
(``"architecture": "<name>"``) load into :class:`HybridLM` and run on
:class:`HybridEngine`. Both engines expose the same ``generate`` call, so
the server, the batcher and the command line do not care which one they
hold.
"""

from __future__ import annotations

import json
import os
from typing import Optional

import torch

# design name -> (checkpoint loader, named tiny/bench specs)
_HYBRID_DESIGNS = {}


def register_hybrid_design(name: str, loader) -> None:
    _HYBRID_DESIGNS[name.lower()] = loader


def _read_config(path: str) -> Optional[dict]:
    cfg = os.path.join(path, "config.json")
    if os.path.isdir(path) and os.path.exists(cfg):
        with open(cfg) as f:
            return json.load(f)
    return None


def hybrid_design_of(path: str) -> Optional[str]:
    """The layer-list design a checkpoint directory names, or None."""
    cfg = _read_config(path)
    arch = (cfg or {}).get("architecture")
    if isinstance(arch, str) and arch.lower() in _HYBRID_DESIGNS:
        return arch.lower()
    return None


def load_model_and_engine(path_or_name: str, engine_cfg, dtype=None,
                          device=None, seed: int = 0):
    """Build (model, engine) for a checkpoint directory or a known model
    name. ``dtype`` None picks bf16 on GPU and fp32 on CPU."""
    if device is None:
        device = torch.device("cuda:0" if torch.cuda.is_available() else "cpu")
    if dtype is None:
        dtype = torch.bfloat16 if device.type == "cuda" else torch.float32
    design = hybrid_design_of(path_or_name)
    if design is not None:
        from ..engine.hybrid_engine import HybridEngine
        model = _HYBRID_DESIGNS[design](path_or_name, dtype=dtype, device=device)
        return model, HybridEngine(model, engine_cfg, device=device, seed=seed)
    cfg = _read_config(path_or_name)
    if cfg is not None and "architecture" in cfg and "architectures" not in cfg:
        raise ValueError(f"unknown model design {cfg['architecture']!r}; "
                         f"known: {sorted(_HYBRID_DESIGNS)}")
    from ..engine.engine import Engine
    from .hf_io import is_hf_checkpoint_dir, load_hf_checkpoint, resolve_spec
    from .model import CausalLM
    model = CausalLM(resolve_spec(path_or_name), dtype=dtype, device=device)
    model.random_init(seed)
    if is_hf_checkpoint_dir(path_or_name):
        load_hf_checkpoint(model, path_or_name)
    return model, Engine(model, engine_cfg, device=device, seed=seed)


def _register_builtin():
    from .hybrid import (load_kakilorn_checkpoint, load_legilix_checkpoint,
                         load_nedasun_checkpoint, load_nibalix_checkpoint)
    register_hybrid_design("Nibalix", load_nibalix_checkpoint)
    register_hybrid_design("Nedasun", load_nedasun_checkpoint)
    register_hybrid_design("Kakilorn", load_kakilorn_checkpoint)
    register_hybrid_design("Legilix", load_legilix_checkpoint)


_register_builtin()

"""Model registry of the serving path: the ``architecture`` entry of a model folder's ``config.json`` picks the loader.

A loader takes ``(model_dir, act_dtype, device)`` and returns a model that serves ragged batches: ``new_cache(device, max_tokens)``, ``step(SeqStep, ...)``
and ``vocab_size`` (what ``generate.RaggedBatch`` drives).  Other designs register themselves with ``register``.
"""

import json
import os

import torch

_LOADERS = {}

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def register(architecture, loader):
    _LOADERS[architecture] = loader


def architectures():
    return sorted(_LOADERS)


def _gemepel(model_dir, act_dtype, device):
    from llm_quest_amd.gemepel.gemepel_weight_loading import load_gemepel

    return load_gemepel(model_dir, act_dtype, device)


def _mepatar(model_dir, act_dtype, device):
    from llm_quest_amd.mepatar.mepatar_weight_loading import load_mepatar

    return load_mepatar(model_dir, act_dtype, device)


def _mopalorn(model_dir, act_dtype, device):
    from llm_quest_amd.mopalorn.mopalorn_weight_loading import load_mopalorn

    return load_mopalorn(model_dir, act_dtype, device)


def _gepilix(model_dir, act_dtype, device):
    from llm_quest_amd.gepilix.gepilix_weight_loading import load_gepilix

    return load_gepilix(model_dir, act_dtype, device)


register("Gemepel", _gemepel)
register("Mepatar", _mepatar)
register("Mopalorn", _mopalorn)
register("Gepilix", _gepilix)


def load_model(model_dir, dtype="bfloat16", device="cuda"):
    """The model of ``model_dir`` (config.json + model.safetensors), chosen by the config's ``architecture``."""
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    arch = cfg.get("architecture") or (cfg.get("architectures") or [None])[0]
    if arch not in _LOADERS:
        raise KeyError(f"no serving model registered for architecture {arch!r} (known: {architectures()})")
    act = DTYPES[dtype] if isinstance(dtype, str) else dtype
    return _LOADERS[arch](model_dir, act, device)

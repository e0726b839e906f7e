"""Configuration of the sparse-attention path.

Mirrors ``kernels/sparse_attn/sparse_attn_config.py`` of the reference for the ``attn``
section only (``GLOBAL_CONFIG`` dict, ``get_kernel_config_attn``, YAML deep-merge loader,
reference lines 4-72, 82-98, 100-131).  There is one provider, ``'hip'``.
"""
from __future__ import annotations

import copy
from typing import Any, Dict

BASE_CONFIG: Dict[str, Any] = {
    "world_size": 1,
    "attn": {
        "is_enabled": True,
        "decision_scale": 10,
        "speedup": 1,
        "top_keys": 0.05,
        "attn_sink": 5,
        "win_size": [-1, -1, -1, -1, -1, -1, -1, -1, 1, 1, 3, 5, 7],
        "cs4a_ws": [1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 7, 9],
        "bound_layer": 10,
        "provider": "hip",
    },
}

GLOBAL_CONFIG: Dict[str, Any] = copy.deepcopy(BASE_CONFIG)


def get_kernel_config_attn() -> Dict[str, int]:
    """Kernel constants (reference ``get_kernel_config_attn``, sparse_attn_config.py:82-98).

    ``bm``: query rows sharing one key list; ``counts_multiple_of``: list lengths are rounded
    to this (one 64-key tile); ``indices_pad_to``: no stride padding is needed.
    The reference providers ``'triton'`` / ``'cuda'`` are accepted as aliases so that a shipped
    YAML (``provider: cuda``) loads unchanged; they select the same HIP kernels and keep the
    reference's list-length granularity for that provider.
    """
    provider = GLOBAL_CONFIG["attn"]["provider"]
    if provider in ("hip", "triton"):
        return {"bm": 192, "counts_multiple_of": 64, "indices_pad_to": 1}
    if provider == "cuda":
        return {"bm": 192, "counts_multiple_of": 112, "indices_pad_to": 4}
    raise ValueError(f"Invalid provider: {provider}")


def update_global_config(config: Dict[str, Any]) -> None:
    GLOBAL_CONFIG.update({**GLOBAL_CONFIG, **config})


def _deep_update(d: Dict[str, Any], u: Dict[str, Any]) -> None:
    for k, v in u.items():
        if isinstance(v, dict) and isinstance(d.get(k), dict):
            _deep_update(d[k], v)
        else:
            d[k] = v


def load_from_file(config_file: str) -> None:
    import yaml

    with open(config_file, "r") as f:
        cfg = yaml.safe_load(f)
    if cfg:
        _deep_update(GLOBAL_CONFIG, cfg)


def reset() -> None:
    GLOBAL_CONFIG.clear()
    GLOBAL_CONFIG.update(copy.deepcopy(BASE_CONFIG))

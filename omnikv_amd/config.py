"""Config object with the reference's `.get(key, default)` behaviour.

modeling/omnikv_config.py:10-23: a missing key is SET to the default (with a
warning) and the default returned, so later reads see the same value.
"""
from __future__ import annotations

import json
import logging
from typing import Any

logger = logging.getLogger("omnikv_amd")

# keys the selection path reads, with the defaults the reference's code uses
PATH_DEFAULTS = {
    "model_cls": "multi",
    "cache_cls": "default",          # modeling/spec_cache.py:836
    "do_select_layers": None,        # required, e.g. "2,8,18"
    "num_wait_load_layers": 2,       # modeling/omnikv.py:333-335
    "real_offload": True,            # modeling/omnikv.py:336
    "dense_more": False,             # must be true: modeling/omnikv.py:211-214
    "num_of_selected_tokens": 4096,  # modeling/omnikv.py:169
    "selector_cls": "softmax_before_last",  # modeling/omnikv.py:138
    "window_size": 16,               # modeling/omnikv.py:139
    "pretraining_tp": -1,
}


class OmniKVConfig:
    """Flat attribute bag; JSON keys are merged on with setattr as infer.py:197-200 does."""

    def __init__(self, **kwargs: Any):
        for k, v in kwargs.items():
            setattr(self, k, v)

    @classmethod
    def from_json(cls, path: str, **overrides: Any) -> "OmniKVConfig":
        with open(path) as f:
            d = json.load(f)
        d.update(overrides)
        return cls(**d)

    def get(self, key: str, default: Any = None) -> Any:
        if hasattr(self, key):
            return getattr(self, key)
        logger.warning("%s not set in config; using default %r", key, default)
        setattr(self, key, default)
        return default

    def set_config(self, **kwargs: Any) -> None:
        for k, v in kwargs.items():
            setattr(self, k, v)

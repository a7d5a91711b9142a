"""Import-path alias: `from attention_variants.causal import attention_pytorch_causal` (the reference's import
path, e.g. its tests/test_causal.py:9) resolves to the MI355X implementation in flashlight_amd.attention_variants."""
import importlib
import sys

from flashlight_amd.attention_variants import *  # noqa: F401,F403

for _name in ("vanilla", "causal", "alibi", "softcap", "sliding_window", "prefix_lm", "document_mask", "diff_attn",
              "evoformer"):
    _mod = importlib.import_module(f"flashlight_amd.attention_variants.{_name}")
    sys.modules[f"{__name__}.{_name}"] = _mod
    globals()[_name] = _mod
del _name, _mod

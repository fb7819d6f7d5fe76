"""Repo-root alias of the drop-in module so that `from flash_tt_attn import attention` works from a
checkout, exactly like the upstream single-file layout (example_usage.py:2).  The implementation
lives in flash-triangle-attention_amd/flash_tt_attn.py."""
import importlib.util as _ilu
import os as _os
import sys as _sys

_pkg = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "flash-triangle-attention_amd")
if _pkg not in _sys.path:
    _sys.path.insert(0, _pkg)
_spec = _ilu.spec_from_file_location("_fta_flash_tt_attn_impl", _os.path.join(_pkg, "flash_tt_attn.py"))
_impl = _ilu.module_from_spec(_spec)
_spec.loader.exec_module(_impl)

attention = _impl.attention
_attention = _impl._attention
reference_tt_attn = _impl.reference_tt_attn
SUPPORTED_HEAD_DIMS = _impl.SUPPORTED_HEAD_DIMS
__all__ = ["attention", "_attention", "reference_tt_attn", "SUPPORTED_HEAD_DIMS"]

"""MI355X-native float8 linear path with the API of lingua/float8.py."""
from .float8 import (  # noqa: F401
    EPS,
    Fp8Linear,
    Fp8LinearFn,
    clear_cast_memos,
    config,
    convert_linears_to_fp8,
    get_scale_rule,
    matmul,
    named_replace,
    scale,
    set_scale_rule,
)

__all__ = [
    "EPS",
    "Fp8Linear",
    "Fp8LinearFn",
    "clear_cast_memos",
    "config",
    "convert_linears_to_fp8",
    "get_scale_rule",
    "matmul",
    "named_replace",
    "scale",
    "set_scale_rule",
]

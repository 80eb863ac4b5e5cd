"""dtype vocabulary of the IR (counterpart of python/aitemplate/compiler/dtype.py)."""

_ALIASES = {"half": "float16", "fp16": "float16", "bf16": "bfloat16", "float": "float32", "fp32": "float32",
            "int": "int32"}
_SIZES = {"float16": 2, "bfloat16": 2, "float32": 4, "int32": 4, "int64": 8, "bool": 1}
# AITemplateDtype enum values of the C ABI (static/include/model_interface.h)
_ENUM = {"float16": 1, "float32": 2, "int32": 3, "int64": 4, "bool": 5, "bfloat16": 6}
_ENUM_NAME = {"float16": "kHalf", "float32": "kFloat", "int32": "kInt", "int64": "kLong", "bool": "kBool",
              "bfloat16": "kBFloat16"}


def normalize_dtype(dtype: str) -> str:
    d = _ALIASES.get(dtype, dtype)
    if d not in _SIZES:
        raise KeyError(f"unknown dtype {dtype}")
    return d


def get_dtype_size(dtype: str) -> int:
    return _SIZES[normalize_dtype(dtype)]


def is_same_dtype(a: str, b: str) -> bool:
    return normalize_dtype(a) == normalize_dtype(b)


def dtype_to_enumerator(dtype: str) -> str:
    return "AITemplateDtype::" + _ENUM_NAME[normalize_dtype(dtype)]


def dtype_enum_value(dtype: str) -> int:
    return _ENUM[normalize_dtype(dtype)]


def dtype_str_to_enum(dtype: str) -> int:
    return dtype_enum_value(dtype)

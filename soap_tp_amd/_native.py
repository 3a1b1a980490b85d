"""ctypes loader for ``libsoap_mi355.so`` (the gfx950 kernels behind a C ABI).

There is deliberately no fallback: if the library has not been built, or a call fails,
an exception is raised.  Error codes are mapped the way the reference's pybind11 modules map
C++ exceptions: ``std::invalid_argument`` -> ``ValueError``, ``std::runtime_error`` ->
``RuntimeError`` (src/soap_tp/csrc/slate_bindings.cpp:69-75, elpa_bindings.cpp:77-91).
"""
from __future__ import annotations

import ctypes
import re
from pathlib import Path
from typing import Dict, List, Tuple

PACKAGE_DIR = Path(__file__).resolve().parent
LIBRARY_PATH = PACKAGE_DIR / "libsoap_mi355.so"
HEADER_PATH = PACKAGE_DIR.parent / "include" / "soap_mi355.h"

OK = 0
INVALID_ARGUMENT = -1
RUNTIME_ERROR = -2
NOT_CONVERGED = -3
WORKSPACE_TOO_SMALL = -4

_C_TYPES = {
    "int": ctypes.c_int,
    "int64_t": ctypes.c_int64,
    "size_t": ctypes.c_size_t,
    "float": ctypes.c_float,
    "double": ctypes.c_double,
    "void": None,
}

_library = None
_signatures: Dict[str, Tuple[object, List[object]]] = {}


def declared_functions(header_text: str | None = None) -> Dict[str, Tuple[str, List[str]]]:
    """Parse ``include/soap_mi355.h`` into {name: (return type, [parameter types])}."""
    if header_text is None:
        header_text = HEADER_PATH.read_text()
    text = re.sub(r"/\*.*?\*/", "", header_text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    functions: Dict[str, Tuple[str, List[str]]] = {}
    pattern = re.compile(r"([A-Za-z_][\w\s\*]*?)\b(soapmi_\w+)\s*\(([^)]*)\)\s*;", re.S)
    for match in pattern.finditer(text):
        return_type = " ".join(match.group(1).split())
        name = match.group(2)
        parameters = []
        raw = match.group(3).strip()
        if raw and raw != "void":
            for parameter in raw.split(","):
                tokens = parameter.strip()
                # drop the parameter name (last identifier), keep type and pointer stars
                tokens = re.sub(r"\b[A-Za-z_]\w*$", "", tokens).strip() if not tokens.endswith("*") else tokens
                parameters.append(" ".join(tokens.split()))
        functions[name] = (return_type, parameters)
    return functions


def _ctype_of(type_text: str):
    if "*" in type_text:
        if "char" in type_text:
            return ctypes.c_char_p
        return ctypes.c_void_p
    base = type_text.replace("const", "").strip()
    if base not in _C_TYPES:
        raise RuntimeError(f"unsupported C type in header: {type_text!r}")
    return _C_TYPES[base]


def library() -> ctypes.CDLL:
    """Load the shared library once and attach ctypes signatures from the header."""
    global _library
    if _library is not None:
        return _library
    if not LIBRARY_PATH.exists():
        raise RuntimeError(
            f"{LIBRARY_PATH} is missing: build the gfx950 kernels first "
            "(python -m soap_tp_amd.build). There is no CPU fallback."
        )
    lib = ctypes.CDLL(str(LIBRARY_PATH))
    for name, (return_type, parameters) in declared_functions().items():
        function = getattr(lib, name)
        function.restype = _ctype_of(return_type)
        function.argtypes = [_ctype_of(parameter) for parameter in parameters]
        _signatures[name] = (function.restype, function.argtypes)
    _library = lib
    return lib


def last_error() -> str:
    return library().soapmi_last_error().decode("utf-8", "replace")


def check(code: int) -> None:
    """Raise the Python exception that corresponds to a negative status code."""
    if code == OK:
        return
    message = last_error()
    if code in (INVALID_ARGUMENT, WORKSPACE_TOO_SMALL):
        raise ValueError(message)
    raise RuntimeError(message or f"libsoap_mi355 returned status {code}")


def call(name: str, *arguments) -> None:
    """Call an int-returning entry point and raise on failure."""
    check(getattr(library(), name)(*arguments))


def device_error_flag(clear: bool = True) -> bool:
    """True if a factorisation that has finished on the current device failed on the device since
    the flag was last cleared (its output is NaN-poisoned).  Does not synchronise."""
    code = library().soapmi_device_error_flag(1 if clear else 0)
    if code < 0:
        check(code)
    return code > 0


def compiled_gpu_backend() -> str:
    return library().soapmi_compiled_gpu_backend().decode()


def world_rank_and_size() -> Tuple[int, int]:
    rank = ctypes.c_int(-1)
    size = ctypes.c_int(-1)
    library().soapmi_world_rank_and_size(ctypes.byref(rank), ctypes.byref(size))
    return rank.value, size.value

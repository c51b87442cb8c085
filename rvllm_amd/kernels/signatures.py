"""The argument types of the kernel library's entry points, read from their declarations in ``csrc/``.

With the types declared, a foreign call takes plain Python numbers (an address as an int, a float as a float) and
converts them itself, which costs a third less host time a launch than building a ``ctypes`` object for every
argument; and an address can no longer be cut to 32 bits by a call that forgot to wrap it, since a function
without a declared signature is refused (``Library.__getattr__``).
"""

from __future__ import annotations

import ctypes
import pathlib
import re

_DECLARATION = re.compile(r'extern\s+"C"\s+([\w\s\*]+?)\s*\b(\w+)\s*\(([^)]*)\)')
_DEFINE = re.compile(r"^\s*#define\s+(\w+)\s+(\w+)\s*$", re.M)
_COMMENT = re.compile(r"//[^\n]*|/\*.*?\*/", re.S)


class SignatureError(RuntimeError):
    pass


def _ctype(text: str, what: str):
    """The ctypes type of one C parameter or return type (the parameter's name, if any, is still on it)."""
    t = re.sub(r"\b(const|__restrict__|volatile|struct)\b", " ", text).strip()
    if "*" in t:
        return ctypes.c_char_p if re.fullmatch(r"char\s*\*", t) and what == "return" else ctypes.c_void_p
    words = t.split()
    if what == "parameter" and len(words) > 1:
        words = words[:-1]  # the name
    kind = " ".join(words)
    known = {"int": ctypes.c_int, "unsigned": ctypes.c_uint, "unsigned int": ctypes.c_uint,
             "long long": ctypes.c_longlong, "unsigned long long": ctypes.c_ulonglong, "size_t": ctypes.c_size_t,
             "float": ctypes.c_float, "double": ctypes.c_double, "bool": ctypes.c_bool,
             "hipStream_t": ctypes.c_void_p, "void": None}
    if kind not in known:
        raise SignatureError(f"unknown C type {text.strip()!r} in a {what}")
    return known[kind]


def read_signatures(csrc: pathlib.Path) -> dict:
    """{entry point: (return type, [argument types])} of every ``extern "C"`` function defined under ``csrc``.
    A function whose name is a macro (one source compiled several times under other names) is listed under every
    name that a ``#define`` of a source gives the macro."""
    defines: dict = {}
    declared = []
    for path in sorted(csrc.iterdir()):
        if path.suffix not in (".hip", ".inc", ".h"):
            continue
        text = _COMMENT.sub(" ", path.read_text())
        for macro, value in _DEFINE.findall(text):
            defines.setdefault(macro, set()).add(value)
        for ret, name, params in _DECLARATION.findall(text):
            declared.append((ret, name, params, path.name))
    table: dict = {}
    for ret, name, params, where in declared:
        params = params.strip()
        pieces = [] if params in ("", "void") else [p for p in params.split(",")]
        try:
            signature = (_ctype(ret, "return"), [_ctype(p, "parameter") for p in pieces])
        except SignatureError as e:
            raise SignatureError(f"{where}: {name}: {e}") from None
        for real in sorted(defines.get(name, {name})):
            if real in table and table[real] != signature:
                raise SignatureError(f"{real} is declared twice with different arguments")
            table[real] = signature
    return table


class Library:
    """The loaded library with every entry point's types set: ``lib.rv_name(...)`` as with ``ctypes.CDLL``, but a
    name without a declaration in the sources is an error instead of a call with guessed types."""

    def __init__(self, cdll: ctypes.CDLL, table: dict):
        self._cdll = cdll
        self._table = table
        self._name = cdll._name

    def __getattr__(self, name: str):
        if name.startswith("_"):
            raise AttributeError(name)
        if name not in self._table:
            raise SignatureError(f"{name} has no declaration in csrc/: its arguments' types are unknown")
        fn = getattr(self._cdll, name)
        fn.restype, fn.argtypes = self._table[name]
        self.__dict__[name] = fn  # found at once from now on
        return fn

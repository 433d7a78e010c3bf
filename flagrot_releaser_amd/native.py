"""One loader for the package's gfx950 shared libraries (libflagrot_kernels / _kivi / _mq .so).

A `Library` knows where its .so lives (in-tree under lib/, or the path an environment variable names), brings it up to
date before the first use (hipcc through flagrot_releaser_amd.build, one builder at a time across processes), checks the
ABI number the library reports against the one the front end was written for, and types every entry point from a compact
signature string.  Calls go through `Library.run`, which takes tensors as they are (their device pointer is passed),
and turns a non-zero status into a RuntimeError carrying the library's own message.  Nothing here computes: without the
library there is no result, and a missing compiler or a failed build is an error, never a fallback.

Signature letters: p pointer (tensor, int or None), i int, l long long, f float.  Every entry point returns int unless
the table says otherwise ("->s": C string).
"""
from __future__ import annotations

import ctypes
import fcntl
import os
from pathlib import Path

import torch

from . import build as _build

_CTYPE = {"p": ctypes.c_void_p, "i": ctypes.c_int, "l": ctypes.c_longlong, "f": ctypes.c_float}


def as_arg(a):
    """what ctypes gets for one Python argument: tensors -> device address, flags -> int, the rest unchanged"""
    if isinstance(a, torch.Tensor):
        return a.data_ptr()
    if isinstance(a, bool):
        return int(a)
    return a


def current_stream() -> int:
    """the raw hipStream_t torch would launch on right now (of the current device)"""
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())


class Library:
    def __init__(self, key: str, env: str, version_fn: str, abi: int, error_fn: str, table: dict):
        """key: name of the library in flagrot_releaser_amd.build; env: variable that may name another .so (then it is
        never rebuilt); table: entry point -> signature string."""
        self.key, self.env, self.version_fn, self.abi, self.error_fn, self.table = key, env, version_fn, abi, error_fn, table
        self._dll = None

    # -------------------------------------------------------------------------------------------- where, and how fresh
    @property
    def path(self) -> Path:
        return Path(os.environ.get(self.env) or _build.lib_path(self.key))

    def _frozen(self) -> bool:
        return bool(os.environ.get("FLAGROT_NO_REBUILD")) or self.env in os.environ

    def _needs_build(self) -> bool:
        so = self.path
        if not so.exists():
            return True
        if self._frozen():
            return False
        built = so.stat().st_mtime
        return any(src.exists() and src.stat().st_mtime > built for src in _build.sources(self.key))

    def _bring_up_to_date(self):
        if not self._needs_build():
            return
        so = self.path
        if self._frozen():
            raise RuntimeError(f"{so} is missing and rebuilding is switched off ({self.env} / FLAGROT_NO_REBUILD)")
        so.parent.mkdir(parents=True, exist_ok=True)
        with open(f"{so}.lock", "w") as gate:
            fcntl.flock(gate, fcntl.LOCK_EX)                      # another process may be building the same file
            try:
                if self._needs_build():
                    _build.build(self.key, verbose=False)
            finally:
                fcntl.flock(gate, fcntl.LOCK_UN)

    # -------------------------------------------------------------------------------------------- the handle
    @property
    def dll(self) -> ctypes.CDLL:
        if self._dll is None:
            self._bring_up_to_date()
            dll = ctypes.CDLL(str(self.path))
            version = getattr(dll, self.version_fn)
            version.restype, version.argtypes = ctypes.c_int, []
            if version() != self.abi:
                raise RuntimeError(f"{self.path.name}: ABI {version()}, this front end speaks {self.abi}; rebuild {self.path}")
            for name, sig in self.table.items():
                fn = getattr(dll, name)
                args, _, ret = sig.partition("->")
                fn.argtypes = [_CTYPE[c] for c in args.split()]
                fn.restype = ctypes.c_char_p if ret.strip() == "s" else ctypes.c_int
            self._dll = dll
        return self._dll

    @property
    def exports(self) -> tuple:
        return (self.version_fn,) + tuple(self.table)

    def last_error(self) -> str:
        return getattr(self.dll, self.error_fn)().decode()

    def ask(self, name: str, *args) -> int:
        """an entry point whose int result is an answer (sizes, counts), not a status"""
        return getattr(self.dll, name)(*map(as_arg, args))

    def run(self, name: str, *args) -> None:
        """an entry point whose int result is a status: 0, or an error this raises with the library's message"""
        status = getattr(self.dll, name)(*map(as_arg, args))
        if status:
            raise RuntimeError(f"{name}: launch failed (code {status}, {self.last_error()})")

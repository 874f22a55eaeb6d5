"""Discovery of the compiled megakernel entry point.

Same contract as reference ``megakernels/mk.py:5-17``: ``mk_dir`` is put on
``sys.path`` and must contain an importable module ``mk_llama`` exposing a
callable ``mk_llama``.  The default directory is this package's ``csrc``,
whose ``mk_llama.py`` binds the C-ABI of ``libmk_llama.so`` (the HIP build for
gfx950).  There is no CPU fallback: a missing library raises.
"""

from __future__ import annotations

import importlib
import sys
from pathlib import Path

DEFAULT_MK_DIR = Path(__file__).parent / "csrc"


def get_mk_module(mk_dir: Path | str | None = None):
    mk_dir = Path(mk_dir) if mk_dir is not None else DEFAULT_MK_DIR
    path = str(mk_dir.expanduser().absolute())
    if path not in sys.path:
        sys.path.append(path)
    return importlib.import_module("mk_llama")


def get_mk_func(mk_dir: Path | str | None = None):
    return get_mk_module(mk_dir).mk_llama


class MK_Interpreter:
    def __init__(self, mk_dir: Path | str | None = None):
        self.mk_module = get_mk_module(mk_dir)
        self.mk_func = self.mk_module.mk_llama

    def interpret(self, globs):
        raise NotImplementedError

    def check_status(self, device=None):
        """Synchronise and raise ``RuntimeError`` if the most recent launch on ``device`` gave up (a
        dependency wait ran out, a malformed instruction, a token outside the vocabulary): its
        outputs are then garbage.  The reference's kernel traps or hangs in these cases
        (``include/util.cuh:38``); this one records a status that has to be looked at.  A module in
        ``mk_dir`` without ``check_status`` is taken to report its own failures."""
        check = getattr(self.mk_module, "check_status", None)
        if check is not None:
            check(device)

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


def get_mk_func(mk_dir: Path | str | None = None):
    mk_dir = Path(mk_dir) if mk_dir is not None else DEFAULT_MK_DIR
    path = str(mk_dir.expanduser().absolute())
    if path not in sys.path:
        sys.path.append(path)
    module = importlib.import_module("mk_llama")
    return module.mk_llama


class MK_Interpreter:
    def __init__(self, mk_dir: Path | str | None = None):
        self.mk_func = get_mk_func(mk_dir)

    def interpret(self, globs):
        raise NotImplementedError

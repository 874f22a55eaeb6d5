"""Writes tests/golden/dot2_vectors.npz: operands and results of the gfx950 instruction V_DOT2_F32_BF16.

Run on a machine with an MI355X from the repository root (the HIP library must be built):

    python tests/golden/make_dot2_vectors.py

The results come from the instruction itself (through the library's self-test entry point), never from the
definition in oracle/exact_math.h: the CPU test suite checks the definition against this file.
"""
import ctypes
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT / "tests"))
import dot2_cases  # noqa: E402

PER_CLASS = 6000


def run_instruction(lib, a, b, acc):
    dev = torch.device("cuda:0")
    ta, tb, tc = (torch.from_numpy(x.astype(np.uint32).view(np.int32)).to(dev) for x in (a, b, acc))
    out = torch.empty_like(ta)
    rc = lib.mk_llama_selftest_dot2(ctypes.c_void_p(ta.data_ptr()), ctypes.c_void_p(tb.data_ptr()), ctypes.c_void_p(tc.data_ptr()),
                                    ctypes.c_void_p(out.data_ptr()), ctypes.c_uint64(ta.numel()),
                                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, rc
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint32)


def main():
    lib = ctypes.CDLL(str(ROOT / "megakernels_amd" / "csrc" / "libmk_llama.so"))
    rng = np.random.default_rng(20240229)
    a, b, acc, names = [], [], [], []
    for gen in dot2_cases.CLASSES:
        x, y, z = gen(rng, PER_CLASS)
        a.append(x.astype(np.uint32)); b.append(y.astype(np.uint32)); acc.append(z.astype(np.uint32))
        names += [gen.__name__] * PER_CLASS
    a, b, acc = np.concatenate(a), np.concatenate(b), np.concatenate(acc)
    out = run_instruction(lib, a, b, acc)
    path = ROOT / "tests" / "golden" / "dot2_vectors.npz"
    np.savez_compressed(path, a=a, b=b, acc=acc, out=out, classes=np.array([g.__name__ for g in dot2_cases.CLASSES]), per_class=PER_CLASS)
    print(f"wrote {path}: {len(a)} cases")


if __name__ == "__main__":
    main()

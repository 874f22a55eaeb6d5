"""The written-out definition of the two-element bf16 dot product (oracle/exact_math.h) against the
instruction itself, through the C ABI: the matvec dot products of the kernel are chains of this
instruction, so the checker's arithmetic is only as good as this agreement."""
import ctypes
import os

import numpy as np
import pytest
import torch

import dot2_cases
from oracle import pyvm

from megakernels_amd.csrc import mk_llama as mk_mod

pytestmark = pytest.mark.gpu


def _instruction(lib, a, b, acc):
    dev = torch.device("cuda:0")
    ta, tb, tc = (torch.from_numpy(np.ascontiguousarray(x, dtype=np.uint32).view(np.int32)).to(dev) for x in (a, b, acc))
    out = torch.empty_like(ta)
    rc = lib.mk_llama_selftest_dot2(ctypes.c_void_p(ta.data_ptr()), ctypes.c_void_p(tb.data_ptr()), ctypes.c_void_p(tc.data_ptr()),
                                    ctypes.c_void_p(out.data_ptr()), ctypes.c_uint64(ta.numel()),
                                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint32)


@pytest.mark.parametrize("gen", dot2_cases.CLASSES, ids=lambda g: g.__name__)
def test_definition_equals_instruction(gen):
    lib = mk_mod.load_library()
    # 11 classes x 5 x 4M: 2.3e8 cases by default; MK_DOT2_ROUNDS widens the search (100: 4.6e9 cases, minutes),
    # MK_DOT2_SEED moves it to other cases
    n, rounds = 1 << 22, int(os.environ.get("MK_DOT2_ROUNDS", "5"))
    seed = int(os.environ.get("MK_DOT2_SEED", "0"))
    for r in range(rounds):
        rng = np.random.default_rng([seed, r, dot2_cases.CLASSES.index(gen)])
        a, b, acc = (np.ascontiguousarray(x, dtype=np.uint32) for x in gen(rng, n))
        hw = _instruction(lib, a, b, acc)
        want = pyvm.dot2(a, b, acc.view(np.float32)).view(np.uint32)
        bad = np.flatnonzero(~dot2_cases.same_results(want, hw))
        assert bad.size == 0, [(hex(a[i]), hex(b[i]), hex(acc[i]), hex(hw[i]), hex(want[i])) for i in bad[:5]]
        if gen is not dot2_cases.any_bits:
            assert not np.any(hw == 0x80000000), "a zero result is +0"


def test_chains_as_the_kernel_runs_them():
    """accumulator chains of the length and operand statistics of a real matvec: each step's input is the
    instruction's own previous result"""
    lib = mk_mod.load_library()
    rng = np.random.default_rng(5)
    n = 1 << 20
    acc_hw = np.zeros(n, dtype=np.uint32)
    acc_def = np.zeros(n, dtype=np.uint32)
    for _ in range(16):
        a, b, _ = dot2_cases.realistic(rng, n)
        acc_hw = _instruction(lib, a, b, acc_hw)
        acc_def = pyvm.dot2(a, b, acc_def.view(np.float32)).view(np.uint32)
        assert np.array_equal(acc_hw, acc_def)

"""The C ABI of libmk_llama.so as far as it can be checked without a GPU: the
library loads, exports every function include/mk_llama.h declares, sizes its
workspace sensibly and refuses malformed launches with a message; and the
kernel's scalar math header, compiled for the host, agrees bit for bit with the
checker's own copy (two files, one specification)."""

import ctypes
import re
import subprocess
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "mk_llama.h"
LIB = ROOT / "megakernels_amd" / "csrc" / "libmk_llama.so"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(mk_llama_\w+)\s*\(", text)))


def load():
    if not LIB.exists():
        from megakernels_amd.csrc import build
        build.build()
    return ctypes.CDLL(str(LIB))


def test_header_declares_the_expected_entry_points():
    assert declared_functions() == ["mk_llama_last_error", "mk_llama_launch", "mk_llama_launch_static", "mk_llama_query",
                                    "mk_llama_read_status", "mk_llama_selftest_bf16", "mk_llama_selftest_dot2",
                                    "mk_llama_workspace_bytes"]


def test_library_exports_every_declared_symbol():
    lib = load()
    for name in declared_functions():
        assert getattr(lib, name) is not None


def test_workspace_size_and_static_queries():
    lib = load()
    lib.mk_llama_workspace_bytes.restype = ctypes.c_uint64
    lib.mk_llama_workspace_bytes.argtypes = [ctypes.c_int32] * 4
    small = lib.mk_llama_workspace_bytes(16, 2048, 8192, 2048)
    big = lib.mk_llama_workspace_bytes(32, 4096, 14336, 2048)
    # 1B: status padded to a 128-byte line + 4 copies x 16 shards x 16 layers x 4 counters + 1024 x 2 LM-head
    # maxima + 4 groups x 2048 partial sums as (value, tag) pairs + 16 layers x 2 rows x 48 padded counters + 2048 stamped
    # pairs (query, K row, V row)
    assert small == 4 * (32 + 4 * 16 * 16 * 4 + 2 * 1024 + 2 * 4 * 2048 + 16 * 2 * 48 * 32 + 2 * 2048)
    assert big > small and big < (5 << 18)
    assert lib.mk_llama_workspace_bytes(0, 2048, 8192, 2048) == 0
    assert lib.mk_llama_query(3) == 6                      # ABI version
    assert lib.mk_llama_query(2) == 576                    # 8 consumer waves + 1 controller wave
    assert 80 * 1024 < lib.mk_llama_query(1) <= 160 * 1024  # one workgroup per CU, within gfx950's LDS
    assert lib.mk_llama_query(4) >= 2048
    assert lib.mk_llama_query(99) == -1


def test_launch_refuses_null_arguments_without_touching_a_gpu():
    lib = load()
    lib.mk_llama_last_error.restype = ctypes.c_char_p
    lib.mk_llama_launch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    assert lib.mk_llama_launch(None, None) == -1
    assert b"null" in lib.mk_llama_last_error()
    import sys
    sys.path.insert(0, str(LIB.parent))
    import mk_llama
    args = mk_llama.MkLlamaArgs()  # all pointers null
    assert lib.mk_llama_launch(ctypes.byref(args), None) == -2
    assert b"null device pointer" in lib.mk_llama_last_error()


def test_static_scratch_launch_refuses_shapes_beyond_its_array_before_touching_a_gpu():
    lib = load()
    lib.mk_llama_last_error.restype = ctypes.c_char_p
    lib.mk_llama_workspace_bytes.restype = ctypes.c_uint64
    lib.mk_llama_workspace_bytes.argtypes = [ctypes.c_int32] * 4
    lib.mk_llama_launch_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    assert lib.mk_llama_launch_static(None, None, None) == -1
    import sys
    sys.path.insert(0, str(LIB.parent))
    import mk_llama
    args = mk_llama.MkLlamaArgs()
    args.num_layers, args.hidden_size, args.intermediate_size, args.matvec_reduction_size = 512, 4096, 14336, 2048
    assert lib.mk_llama_workspace_bytes(512, 4096, 14336, 2048) > (2 << 20)
    assert lib.mk_llama_launch_static(ctypes.byref(args), None, None) == -6
    assert b"static scratch" in lib.mk_llama_last_error()
    # every shape the kernel has an instance for fits
    assert lib.mk_llama_workspace_bytes(32, 4096, 14336, 2048) <= (2 << 20)


def test_python_args_struct_matches_the_header():
    """Field order and count of the ctypes mirror follow the C declaration."""
    import sys
    sys.path.insert(0, str(LIB.parent))
    import mk_llama
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    body = text[text.index("typedef struct mk_llama_args {"):text.index("} mk_llama_args;")]
    names = []
    for decl in body.split(";"):
        decl = decl.split("{")[-1].strip()
        if not decl:
            continue
        for part in decl.split(","):
            names.append(re.findall(r"(\w+)\s*$", part.strip())[0])
    assert names == [f[0] for f in mk_llama.MkLlamaArgs._fields_]
    # 23 pointers, pos_id + 2 floats + flag, 14 int shapes, workspace ptr + u64 + 2 x u32, 3 optional pointers
    assert ctypes.sizeof(mk_llama.MkLlamaArgs) == 23 * 8 + 4 * 4 + 14 * 4 + 8 + 8 + 8 + 3 * 8 + 2 * 4


SHIM = r"""
#include "mk_math.h"
extern "C" {
float p_exp(float x) { return mkm::expf_exact(x); }
float p_exp2(float x) { return mkm::exp2f_exact(x); }
float p_log2(float x) { return mkm::log2f_exact(x); }
float p_silu(float x) { return mkm::silu_exact(x); }
unsigned p_bf16(float x) { return mkm::f32_to_bf16(x); }
}
"""


def test_kernel_math_header_equals_checker_math(tmp_path):
    src = tmp_path / "shim.cpp"
    src.write_text(SHIM)
    so = tmp_path / "shim.so"
    subprocess.run(["g++", "-O2", "-shared", "-fPIC", "-mfma", "-ffp-contract=off", "-std=c++17",
                    f"-I{LIB.parent}", str(src), "-o", str(so)], check=True)
    shim = ctypes.CDLL(str(so))
    from oracle import pyvm
    orc = pyvm.load_lib()
    for f in (shim.p_exp, shim.p_exp2, shim.p_log2, shim.p_silu):
        f.argtypes = [ctypes.c_float]
        f.restype = ctypes.c_float
    shim.p_bf16.argtypes = [ctypes.c_float]
    shim.p_bf16.restype = ctypes.c_uint
    rng = np.random.default_rng(3)
    xs = np.concatenate([rng.uniform(-90, 90, 20000), rng.uniform(-1, 1, 5000), [0.0, -0.0, 88.0, -86.0, 1e-30]]).astype(np.float32)
    as_bits = lambda v: np.float32(v).view(np.uint32)
    for x in xs:
        x = float(x)
        assert as_bits(shim.p_exp(x)) == as_bits(orc.mk_oracle_expf(x))
        assert as_bits(shim.p_exp2(x)) == as_bits(orc.mk_oracle_exp2f(x))
        assert shim.p_bf16(x) == orc.mk_oracle_f32_to_bf16(x)
        if x > 0:
            assert as_bits(shim.p_log2(x)) == as_bits(orc.mk_oracle_log2f(x))
    # silu as the checker composes it: g / (1 + exp(-g)) with IEEE division
    for x in xs[:5000]:
        x = np.float32(x)
        want = np.float32(x / np.float32(np.float32(1.0) + np.float32(orc.mk_oracle_expf(float(-x)))))
        assert as_bits(shim.p_silu(float(x))) == as_bits(want)

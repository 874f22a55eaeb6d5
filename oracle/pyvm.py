"""TEST INFRASTRUCTURE: ctypes front end of the C checker (``mk_oracle.c``).

Drives ``libmk_oracle.so`` over the linear instruction list of a schedule,
the way the reference's ``PyVM_Interpreter`` drives its Python solvers
(``megakernels/python_vm.py:83-95``), and provides the token loop of
``megakernels/generators.py:121-163`` on top of it (embedding row, barrier
reset, one VM step, first-maximum argmax over the bf16 logits).

All tensors must live on the CPU and be contiguous; bf16 tensors are handed
to C as their 16-bit patterns.
"""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import torch

from megakernels_amd.scheduler import serialize_and_pad

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libmk_oracle.so"
_lib = None

_U16P = ctypes.POINTER(ctypes.c_uint16)
_F32P = ctypes.POINTER(ctypes.c_float)
_I32P = ctypes.POINTER(ctypes.c_int32)


class _Globals(ctypes.Structure):
    _fields_ = (
        [(n, _U16P) for n in (
            "qkv_proj_weights", "attn_ln_weights", "o_proj_weights", "mlp_ln_weights",
            "up_proj_weights", "gate_proj_weights", "down_proj_weights",
            "lm_head_norm_weights", "lm_head_weights", "k_cache", "v_cache")]
        + [("rope_cos", _F32P), ("rope_sin", _F32P)]
        + [(n, _U16P) for n in ("hidden_states", "post_ln_rope_q", "attn_out")]
        + [("attn_lse_intermediates", _F32P), ("attn_out_intermediates", _F32P)]
        + [("silu_out", _U16P), ("logits", _U16P), ("barriers", _I32P)]
        + [(n, ctypes.c_int32) for n in (
            "num_hidden_layers", "num_attention_heads", "num_kv_heads", "head_dim",
            "hidden_size", "intermediate_size", "vocab_size", "kv_max_len", "max_partials",
            "matvec_reduction_size", "attn_reduction_size", "pos_id", "skip_attn_reduction",
            "check_barriers")]
        + [("attn_scale", ctypes.c_float), ("rms_norm_eps", ctypes.c_float)]
    )


def build(force: bool = False) -> Path:
    """Compile the checker with the Makefile next to it."""
    if force and _LIB_PATH.exists():
        _LIB_PATH.unlink()
    subprocess.run(["make", "-s", "-C", str(_HERE), "libmk_oracle.so"], check=True)
    return _LIB_PATH


def load_lib():
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        lib = ctypes.CDLL(str(_LIB_PATH))
        lib.mk_oracle_run.argtypes = [ctypes.POINTER(_Globals), _I32P, ctypes.c_int]
        lib.mk_oracle_run.restype = ctypes.c_int
        lib.mk_oracle_last_error.restype = ctypes.c_char_p
        lib.mk_oracle_threads.restype = ctypes.c_int
        lib.mk_oracle_argmax_bf16.argtypes = [_U16P, ctypes.c_int]
        lib.mk_oracle_argmax_bf16.restype = ctypes.c_int
        for name in ("mk_oracle_expf", "mk_oracle_exp2f", "mk_oracle_log2f"):
            getattr(lib, name).argtypes = [ctypes.c_float]
            getattr(lib, name).restype = ctypes.c_float
        lib.mk_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        lib.mk_oracle_f32_to_bf16.restype = ctypes.c_uint16
        lib.mk_oracle_dot.argtypes = [_U16P, _F32P, ctypes.c_int]
        lib.mk_oracle_dot.restype = ctypes.c_float
        lib.mk_oracle_dot2.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
        lib.mk_oracle_dot2.restype = None
        lib.mk_oracle_dot2_general.argtypes = lib.mk_oracle_dot2.argtypes
        lib.mk_oracle_dot2_general.restype = None
        _lib = lib
    return _lib


def dot2(a, b, acc, general: bool = False):
    """acc + a.lo * b.lo + a.hi * b.hi per element: numpy uint32 bf16 pairs and float32 accumulators.
    ``general``: through the clause-by-clause form only."""
    import numpy as np

    a = np.ascontiguousarray(a, dtype=np.uint32)
    b = np.ascontiguousarray(b, dtype=np.uint32)
    acc = np.ascontiguousarray(acc, dtype=np.float32)
    out = np.empty_like(acc)
    fn = load_lib().mk_oracle_dot2_general if general else load_lib().mk_oracle_dot2
    fn(a.ctypes.data, b.ctypes.data, acc.ctypes.data, out.ctypes.data, a.size)
    return out


class OracleError(AssertionError):
    """A solver's barrier assertion or argument check failed."""


def _ptr(t: torch.Tensor, ctype, dtype):
    if t.device.type != "cpu":
        raise ValueError("the CPU checker needs CPU tensors")
    if t.dtype != dtype:
        raise TypeError(f"expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError("tensor must be contiguous")
    return ctypes.cast(t.data_ptr(), ctype)


def _pack(globs, check_barriers: bool) -> _Globals:
    bf, f32, i32 = torch.bfloat16, torch.float32, torch.int32
    s = _Globals()
    for name in ("qkv_proj_weights", "attn_ln_weights", "o_proj_weights", "mlp_ln_weights",
                 "up_proj_weights", "gate_proj_weights", "down_proj_weights",
                 "lm_head_norm_weights", "lm_head_weights", "k_cache", "v_cache",
                 "hidden_states", "post_ln_rope_q", "attn_out", "silu_out", "logits"):
        setattr(s, name, _ptr(getattr(globs, name), _U16P, bf))
    for name in ("rope_cos", "rope_sin", "attn_lse_intermediates", "attn_out_intermediates"):
        setattr(s, name, _ptr(getattr(globs, name), _F32P, f32))
    s.barriers = _ptr(globs.barriers, _I32P, i32)
    if globs.k_cache.shape[1] != 1:
        raise ValueError("batch size must be 1")
    s.num_hidden_layers = globs.num_hidden_layers
    s.num_attention_heads = globs.num_attention_heads
    s.num_kv_heads = globs.num_kv_heads
    s.head_dim = globs.head_dim
    s.hidden_size = globs.hidden_size
    s.intermediate_size = globs.intermediate_size
    s.vocab_size = globs.vocab_size
    s.kv_max_len = globs.k_cache.shape[2]
    s.max_partials = globs.attn_lse_intermediates.shape[1]
    s.matvec_reduction_size = globs.matvec_reduction_size
    s.attn_reduction_size = globs.attn_reduction_size
    s.pos_id = int(globs.pos_id)
    s.skip_attn_reduction = int(bool(globs.skip_attn_reduction))
    s.check_barriers = int(check_barriers)
    s.attn_scale = globs.attn_scale
    s.rms_norm_eps = globs.rms_norm_eps
    return s


def words_of(instructions) -> torch.Tensor:
    """``int32 [n, 32]`` word rows for a list of instruction objects (or an
    already tensorised ``[..., 32]`` block, flattened in order)."""
    if isinstance(instructions, torch.Tensor):
        return instructions.reshape(-1, 32).to(torch.int32).cpu().contiguous()
    return torch.tensor([serialize_and_pad(i) for i in instructions], dtype=torch.int32).reshape(-1, 32)


def interpret(globs, instructions, check_barriers: bool = True) -> None:
    """Execute the instructions in order on ``globs`` (in place)."""
    lib = load_lib()
    words = words_of(instructions)
    packed = _pack(globs, check_barriers)
    rc = lib.mk_oracle_run(ctypes.byref(packed), _ptr(words, _I32P, torch.int32), words.shape[0])
    if rc != 0:
        raise OracleError(lib.mk_oracle_last_error().decode())


def argmax_bf16(logits: torch.Tensor) -> int:
    return load_lib().mk_oracle_argmax_bf16(_ptr(logits, _U16P, torch.bfloat16), logits.numel())


def threads() -> int:
    return load_lib().mk_oracle_threads()


class OracleInterpreter:
    """Counterpart of the reference's ``PyVM_Interpreter``."""

    def interpret(self, globs, instructions):
        interpret(globs, instructions)


class OracleGenerator:
    """Greedy decode on the CPU checker.  Tokens are the first-maximum argmax
    of the ``logits`` buffer the LM-head instruction fills, i.e. what the
    megakernel path returns (``generators.py:140-141``)."""

    def __init__(self, model, schedule):
        self.model = model
        self.schedule = schedule
        self.words = words_of(schedule.get_linear_instructions())

    def run(self, token_id: int, pos_id: int) -> int:
        globs = self.schedule.globs
        globs.hidden_states[:] = self.model.model.embed_tokens.weight[token_id]
        globs.barriers.zero_()
        globs.pos_id = pos_id
        interpret(globs, self.words)
        return argmax_bf16(globs.logits)

    def generate(self, output_tokens, prompt_len: int, ntok: int, ntok_already_generated: int = 1):
        for i in range(ntok):
            src = ntok_already_generated + i - 1
            pos_id = prompt_len + ntok_already_generated + i - 1
            output_tokens[0, src + 1] = self.run(int(output_tokens[0, src]), pos_id)

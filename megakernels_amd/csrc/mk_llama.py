"""Python module ``mk_llama`` for ``mk_dir``: binds the C ABI of
``libmk_llama.so`` with ctypes and exposes ``mk_llama(...)`` with the
positional signature the reference's compiled module has
(``megakernels/demos/latency/mk.py:15-49`` calling
``demos/low-latency-llama/llama.cu:26-52``).

PyTorch is used only to read device pointers, shapes and the stream handle,
and to own the small scratch workspace.  There is no fallback: if the library
is missing or a launch is refused, a ``RuntimeError`` is raised.
"""

from __future__ import annotations

import ctypes
from pathlib import Path

import torch

import os

_HERE = Path(__file__).resolve().parent
# MK_LLAMA_LIB selects another build of the same ABI (for comparing kernel variants).  A library that
# is not the one built next to this file is announced on stderr when it is loaded, so that it cannot
# stand in for the product unnoticed.
LIBRARY = Path(os.environ.get("MK_LLAMA_LIB", _HERE / "libmk_llama.so"))

_P = ctypes.c_void_p
_I = ctypes.c_int32
_F = ctypes.c_float


class MkLlamaArgs(ctypes.Structure):
    """``mk_llama_args`` of ``include/mk_llama.h``."""

    _fields_ = (
        [(n, _P) for n in (
            "barriers", "instructions", "timings",
            "qkv_weights", "attn_norm_weights", "o_weights", "mlp_norm_weights",
            "up_weights", "gate_weights", "down_weights", "lm_head_norm_weights", "lm_head_weights",
            "k_cache", "v_cache", "rope_cos", "rope_sin",
            "hidden_states", "q_post_rope", "attn_out", "attn_lse_intermediates",
            "attn_out_intermediates", "silu_out", "logits")]
        + [("pos_id", _I), ("attn_scale", _F), ("rms_norm_eps", _F), ("skip_attn_reduction", _I)]
        + [(n, _I) for n in (
            "num_layers", "hidden_size", "intermediate_size", "num_attention_heads", "num_kv_heads",
            "head_dim", "vocab_size", "num_workers", "num_slots", "kv_max_len", "max_partials",
            "rope_positions", "matvec_reduction_size", "attn_reduction_size")]
        + [("workspace", _P), ("workspace_bytes", ctypes.c_uint64),
           ("spin_limit_us", ctypes.c_uint32), ("flags", ctypes.c_uint32)]
        + [("embed_table", _P), ("token_in", _P), ("token_out", _P)]
        + [("num_steps", _I), ("reserved0", _I)]
    )


_lib = None
_workspaces: dict[tuple, torch.Tensor] = {}

# barrier waits give up after this many microseconds (0 = library default)
spin_limit_us = 0
# set to True to have every launch fill the `timings` tensor (see MK_FLAG_TIMINGS in mk_llama.h)
record_timings = False
# set to True to launch through mk_llama_launch_static: the workspace is then the library's own
# per-GPU array and this module allocates nothing for a launch
static_scratch = False
_static_scratch_ptrs: dict[int, int] = {}
_static_status_pending: dict[int, bool] = {}   # a static launch whose failure, if any, has not been reported yet
# MK_FLAG_JOINT_RESIDUAL for launches that do not say (`joint_residual=` of mk_llama): None = set it
# when the instruction tensor qualifies, False = never (every column-group job runs on its own)
joint_residual_default = None


def load_library():
    global _lib
    if _lib is None:
        if not LIBRARY.exists():
            raise RuntimeError(
                f"{LIBRARY} is missing: build it with `python {_HERE / 'build.py'}` (needs hipcc)"
            )
        if LIBRARY.resolve() != (_HERE / "libmk_llama.so").resolve():
            import sys

            print(f"mk_llama: MK_LLAMA_LIB is set - loading {LIBRARY} instead of {_HERE / 'libmk_llama.so'}", file=sys.stderr)
        lib = ctypes.CDLL(str(LIBRARY))
        lib.mk_llama_launch.argtypes = [ctypes.POINTER(MkLlamaArgs), _P]
        lib.mk_llama_launch.restype = ctypes.c_int
        lib.mk_llama_launch_static.argtypes = [ctypes.POINTER(MkLlamaArgs), _P, ctypes.POINTER(_P)]
        lib.mk_llama_launch_static.restype = ctypes.c_int
        lib.mk_llama_workspace_bytes.argtypes = [_I, _I, _I, _I]
        lib.mk_llama_workspace_bytes.restype = ctypes.c_uint64
        lib.mk_llama_read_status.argtypes = [_P, _P, ctypes.POINTER(_I * 4)]
        lib.mk_llama_read_status.restype = ctypes.c_int
        lib.mk_llama_query.argtypes = [ctypes.c_int]
        lib.mk_llama_query.restype = ctypes.c_int
        lib.mk_llama_last_error.restype = ctypes.c_char_p
        _lib = lib
    return _lib


def _workspace(device: torch.device, num_layers: int, hidden: int, inter: int, reduction: int) -> torch.Tensor:
    key = (device.index, num_layers, hidden, inter, reduction)
    ws = _workspaces.get(key)
    if ws is None:
        nbytes = load_library().mk_llama_workspace_bytes(num_layers, hidden, inter, reduction)
        ws = torch.zeros((nbytes + 3) // 4, dtype=torch.int32, device=device)
        _workspaces[key] = ws
    return ws


def _check(t: torch.Tensor, dtype: torch.dtype, name: str) -> int:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor")
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    return t.data_ptr()


def _token_pointer(t, name, count=1):
    if (not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.int64 or t.numel() != count
            or not t.is_contiguous()):
        raise RuntimeError(f"{name} must be a contiguous int64 device tensor of {count} element(s)")
    return t.data_ptr()


def complete_residual_sets(instructions: torch.Tensor, hidden: int, inter: int, reduction: int) -> bool:
    """Whether the column-group jobs of the residual projections (opcodes 4 and 6) come in complete
    sets: every (opcode, layer, row block) that occurs in ``instructions`` occurs exactly once for
    every column group.  That is what ``MK_FLAG_JOINT_RESIDUAL`` promises the kernel.  The answer is
    kept on the tensor object (and dropped when the tensor is written to)."""
    cached = getattr(instructions, "_mk_complete_residual_sets", None)
    if cached is not None and cached[0] == instructions._version:
        return cached[1]
    words = instructions.detach().cpu().reshape(-1, instructions.shape[-1]).numpy()
    complete = True
    for opcode, in_dim in ((4, hidden), (6, inter)):
        groups = in_dim // reduction
        rows = words[words[:, 0] == opcode]
        if groups <= 1 or len(rows) == 0:
            continue
        seen: dict[tuple[int, int], list[int]] = {}
        for layer, start, end, group in rows[:, 1:5].tolist():
            for block in range(start, end):
                seen.setdefault((layer, block), []).append(group)
        if any(sorted(found) != list(range(groups)) for found in seen.values()):
            complete = False
    instructions._mk_complete_residual_sets = (instructions._version, complete)
    return complete


def mk_llama(
    barriers, instructions, timings,
    qkv_weights, attn_norm_weights, o_weights, mlp_norm_weights,
    up_weights, gate_weights, down_weights, lm_head_norm_weights, lm_head_weights,
    k_cache, v_cache, rope_cos, rope_sin,
    hidden_states, q_post_rope, attn_out, attn_lse_intermediates, attn_out_intermediates,
    silu_out, logits,
    pos_id, attn_scale, rms_norm_eps, skip_attn_reduction,
    stream=None,
    *,
    embed_table=None, token_in=None, token_out=None, reset_barriers=False, num_steps=1,
    joint_residual=None,
):
    """Launch one decode step asynchronously on ``stream`` (a torch stream;
    default: the current one).  Shapes are taken from the tensors.

    The keyword-only arguments fold the glue of the decode loop into the
    launch (no counterpart in the reference binding): ``token_in`` / ``token_out``
    are one-element int64 device tensors (views into the token buffer) - the
    step starts from ``embed_table[token_in]`` instead of ``hidden_states`` and
    writes ``argmax(logits)`` to ``token_out``; ``reset_barriers`` leaves
    ``barriers`` zeroed for the next launch.  ``num_steps`` > 1 runs that many
    decode steps in the one launch: step ``s`` works at position ``pos_id + s``
    from the token of step ``s - 1`` and writes ``token_out[s]`` (``token_out``
    then has ``num_steps`` elements).  ``joint_residual`` sets or clears
    ``MK_FLAG_JOINT_RESIDUAL`` (the column-group jobs of a residual projection
    share their rows instead of exchanging partial sums); by default the
    instruction tensor is inspected once and the flag set when it qualifies."""
    lib = load_library()
    bf, f32, i32 = torch.bfloat16, torch.float32, torch.int32
    a = MkLlamaArgs()
    a.barriers = _check(barriers, i32, "barriers")
    a.instructions = _check(instructions, i32, "instructions")
    a.timings = _check(timings, i32, "timings") if timings is not None else None
    for field, tensor in (
        ("qkv_weights", qkv_weights), ("attn_norm_weights", attn_norm_weights), ("o_weights", o_weights),
        ("mlp_norm_weights", mlp_norm_weights), ("up_weights", up_weights), ("gate_weights", gate_weights),
        ("down_weights", down_weights), ("lm_head_norm_weights", lm_head_norm_weights),
        ("lm_head_weights", lm_head_weights), ("k_cache", k_cache), ("v_cache", v_cache),
        ("hidden_states", hidden_states), ("q_post_rope", q_post_rope), ("attn_out", attn_out),
        ("silu_out", silu_out), ("logits", logits),
    ):
        setattr(a, field, _check(tensor, bf, field))
    for field, tensor in (
        ("rope_cos", rope_cos), ("rope_sin", rope_sin),
        ("attn_lse_intermediates", attn_lse_intermediates), ("attn_out_intermediates", attn_out_intermediates),
    ):
        setattr(a, field, _check(tensor, f32, field))

    if instructions.ndim != 3 or instructions.shape[2] != 32:
        raise RuntimeError("instructions must be [workers, slots, 32]")
    if k_cache.ndim != 4 or k_cache.shape != v_cache.shape:
        raise RuntimeError("k_cache / v_cache must be [(L B), T, KVH, D] of equal shape")
    num_layers, inter, hidden = up_weights.shape
    layers_times_batch, kv_max_len, kv_heads, head_dim = k_cache.shape
    if layers_times_batch != num_layers:
        raise RuntimeError("batch size must be 1")
    heads = attn_lse_intermediates.shape[0]
    if tuple(barriers.shape) != (num_layers, 10, heads + 2 * kv_heads):
        raise RuntimeError(f"barriers must be [{num_layers}, 10, {heads + 2 * kv_heads}]")
    if tuple(qkv_weights.shape) != (num_layers, (heads + 2 * kv_heads) * head_dim, hidden):
        raise RuntimeError("qkv weights do not match [L, (H + 2 KVH) D, hidden]")
    if tuple(o_weights.shape) != (num_layers, hidden, hidden) or tuple(down_weights.shape) != (num_layers, hidden, inter):
        raise RuntimeError("o / down weights have unexpected shapes")
    if tuple(gate_weights.shape) != (num_layers, inter, hidden) or tuple(lm_head_weights.shape[1:]) != (hidden,):
        raise RuntimeError("gate / lm_head weights have unexpected shapes")
    if tuple(rope_cos.shape[1:]) != (head_dim,) or rope_cos.shape != rope_sin.shape:
        raise RuntimeError("rope tables must be [positions, head_dim]")
    if tuple(attn_out_intermediates.shape) != (heads, attn_lse_intermediates.shape[1], head_dim):
        raise RuntimeError("attention intermediates have unexpected shapes")
    for name, tensor, n in (
        ("hidden_states", hidden_states, hidden), ("q_post_rope", q_post_rope, heads * head_dim),
        ("attn_out", attn_out, heads * head_dim), ("silu_out", silu_out, inter),
        ("attn_norm_weights", attn_norm_weights, num_layers * hidden),
        ("mlp_norm_weights", mlp_norm_weights, num_layers * hidden),
        ("lm_head_norm_weights", lm_head_norm_weights, hidden),
    ):
        if tensor.numel() != n:
            raise RuntimeError(f"{name} has {tensor.numel()} elements, expected {n}")
    vocab = lm_head_weights.shape[0]
    if logits.numel() != vocab:
        raise RuntimeError("logits do not match the LM head")

    # column-group width of the residual matvecs: 2048 as in the reference
    # (megakernels/demos/latency/scheduler.py:109); a narrower model is one group
    reduction = min(2048, hidden)

    a.pos_id = int(pos_id)
    a.attn_scale = float(attn_scale)
    a.rms_norm_eps = float(rms_norm_eps)
    a.skip_attn_reduction = int(bool(skip_attn_reduction))
    a.num_layers, a.hidden_size, a.intermediate_size = num_layers, hidden, inter
    a.num_attention_heads, a.num_kv_heads, a.head_dim, a.vocab_size = heads, kv_heads, head_dim, vocab
    a.num_workers, a.num_slots = instructions.shape[0], instructions.shape[1]
    a.kv_max_len = kv_max_len
    a.max_partials = attn_lse_intermediates.shape[1]
    a.rope_positions = rope_cos.shape[0]
    a.matvec_reduction_size = reduction
    a.attn_reduction_size = 4
    if not static_scratch:
        ws = _workspace(barriers.device, num_layers, hidden, inter, reduction)
        a.workspace = ws.data_ptr()
        a.workspace_bytes = ws.numel() * 4
    a.spin_limit_us = int(spin_limit_us)
    if joint_residual is None:
        joint_residual = joint_residual_default
    if joint_residual is None:
        joint_residual = complete_residual_sets(instructions, hidden, inter, reduction)
    a.flags = ((1 if (record_timings and timings is not None) else 0) | (2 if reset_barriers else 0)
               | (4 if joint_residual else 0))
    if token_in is not None:
        if embed_table is None or tuple(embed_table.shape) != (vocab, hidden):
            raise RuntimeError("token_in needs embed_table of shape [vocab, hidden]")
        a.embed_table = _check(embed_table, bf, "embed_table")
        a.token_in = _token_pointer(token_in, "token_in")
    num_steps = int(num_steps)
    if num_steps < 1:
        raise RuntimeError("num_steps must be at least 1")
    if token_out is not None:
        a.token_out = _token_pointer(token_out, "token_out", num_steps)
    a.num_steps = num_steps

    if stream is None:
        stream = torch.cuda.current_stream(barriers.device)
    if static_scratch:
        with torch.cuda.device(barriers.device):
            where = _P()
            rc = lib.mk_llama_launch_static(ctypes.byref(a), ctypes.c_void_p(stream.cuda_stream), ctypes.byref(where))
        if where.value:
            # (every static launch clears the part of the array it uses, status included, so what is
            # read from it afterwards belongs to this launch)
            _static_scratch_ptrs[barriers.device.index] = where.value
            _static_status_pending[barriers.device.index] = True
    else:
        rc = lib.mk_llama_launch(ctypes.byref(a), ctypes.c_void_p(stream.cuda_stream))
    if rc != 0:
        raise RuntimeError(f"mk_llama_launch failed ({rc}): {lib.mk_llama_last_error().decode()}")


STATUS_NAMES = {0: "ok", 1: "barrier wait timed out", 2: "unknown opcode",
                3: "attention partition longer than the on-chip score buffer", 4: "malformed instruction",
                5: "input token outside the vocabulary"}


def read_status(device=None, stream=None):
    """Synchronise and return ``(code, worker, slot, opcode)`` of the most
    recent launch on ``device``.  After a non-zero code the workspace is
    zeroed again so the next launch starts clean."""
    lib = load_library()
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    out = (_I * 4)()
    result = (0, 0, 0, 0)
    if stream is None:
        stream = torch.cuda.current_stream(device)
    for key, ws in _workspaces.items():
        if key[0] != device.index:
            continue
        rc = lib.mk_llama_read_status(ctypes.c_void_p(ws.data_ptr()), ctypes.c_void_p(stream.cuda_stream), ctypes.byref(out))
        if rc != 0:
            raise RuntimeError(f"mk_llama_read_status failed: {lib.mk_llama_last_error().decode()}")
        if out[0] != 0:
            result = tuple(out)
            ws.zero_()
    # the library's own array (launches with static_scratch): every such launch clears what it uses
    # first, so a recorded failure needs no clean-up here
    where = _static_scratch_ptrs.get(device.index)
    if where and _static_status_pending.get(device.index):
        rc = lib.mk_llama_read_status(ctypes.c_void_p(where), ctypes.c_void_p(stream.cuda_stream), ctypes.byref(out))
        if rc != 0:
            raise RuntimeError(f"mk_llama_read_status failed: {lib.mk_llama_last_error().decode()}")
        if out[0] != 0:
            _static_status_pending[device.index] = False   # reported once; the next static launch clears the array
            if result[0] == 0:
                result = tuple(out)
    return result


def check_status(device=None):
    """Raise if the most recent launch recorded an error."""
    code, worker, slot, opcode = read_status(device)
    if code != 0:
        raise RuntimeError(
            f"megakernel gave up: {STATUS_NAMES.get(code, code)} (worker {worker}, slot {slot}, opcode {opcode})"
        )

"""Instruction base types and the buffer bundle shared by every interpreter.

Mirrors the public surface of reference ``megakernels/instructions.py``:

* :class:`BaseGlobals` (``instructions.py:10-69``) - every device buffer the
  virtual machine touches plus the model constants.
* :class:`Instruction` with :meth:`Instruction.serialize`
  (``instructions.py:83-119``) - the word encoding consumed by the device
  interpreter: ``[opcode, field, field, ...]`` in dataclass field order, where an
  ``int`` is one word, a list/tuple is its length followed by its items and
  ``None`` is a single zero.
* :class:`NoOp`, opcode 0 (``instructions.py:122-126``), used to pad queues.

Added here (no counterpart in the reference): :meth:`Instruction.from_words`,
the inverse of ``serialize`` used by tests and by the CPU checker to read back
a tensorised schedule.
"""

from __future__ import annotations

import typing
from dataclasses import dataclass, fields
from typing import Any, ClassVar

from torch import Tensor

from megakernels_amd.model_types import DeviceType
from megakernels_amd.utils import get_sm_count


@dataclass
class BaseGlobals:
    # stacked model parameters: one leading layer dimension
    qkv_proj_weights: Tensor
    attn_ln_weights: Tensor
    o_proj_weights: Tensor
    mlp_ln_weights: Tensor
    up_proj_weights: Tensor
    gate_proj_weights: Tensor
    down_proj_weights: Tensor
    lm_head_norm_weights: Tensor
    lm_head_weights: Tensor
    k_cache: Tensor
    v_cache: Tensor

    # shared by all layers
    rope_cos: Tensor
    rope_sin: Tensor

    # architecture constants
    num_hidden_layers: int
    num_attention_heads: int
    num_kv_heads: int
    head_dim: int
    hidden_size: int
    intermediate_size: int
    vocab_size: int

    attn_scale: float
    rms_norm_eps: float
    device: DeviceType

    hidden_states: Tensor
    barriers: Tensor

    pos_id: int

    def __post_init__(self):
        # filled in by scheduler.tensorize_instructions
        self.instructions: Tensor | None = None
        self.timings: Tensor | None = None

    def sm_count(self) -> int:
        """Worker count the schedule is built for (one workgroup per compute
        unit on MI355X; reference ``instructions.py:51-52``)."""
        return get_sm_count(self.device)

    def num_total_heads(self) -> int:
        return self.num_attention_heads + 2 * self.num_kv_heads

    def mutable_tensor_names(self) -> list[str]:
        """Names of the tensor fields an interpreter may write: everything that
        is not a weight or a rope table (the selection rule of reference
        ``instructions.py:54-66``)."""
        names = []
        for f in fields(self):
            value = getattr(self, f.name)
            if not isinstance(value, Tensor):
                continue
            if "weights" in f.name or f.name in ("rope_cos", "rope_sin"):
                continue
            names.append(f.name)
        return names

    def diff(self, other: "BaseGlobals", skip_kv_cache: bool = False, quiet: bool = False):
        """Compare every mutable tensor with ``other`` and return
        ``{name: (max abs diff, mean rel diff)}``; prints one line per tensor
        unless ``quiet`` (reference ``instructions.py:54-66``)."""
        report = {}
        for name in self.mutable_tensor_names():
            if skip_kv_cache and "cache" in name:
                continue
            _, adiff, rdiff = diff_tensors(
                getattr(self, name), getattr(other, name), name, quiet=quiet
            )
            report[name] = (float(adiff.max()), float(rdiff.mean()))
        return report


def diff_tensors(a: Tensor, b: Tensor, name: str, quiet: bool = False):
    """Absolute and symmetric relative difference of two tensors
    (reference ``instructions.py:72-80``)."""
    a = a.float()
    b = b.float()
    diff = a - b
    adiff = diff.abs()
    rdiff = 2 * adiff / (a.abs() + b.abs() + 1e-6)
    if not quiet:
        print(f"{name}: max adiff: {adiff.max()}, mean rdiff: {rdiff.mean()}")
    return diff, adiff, rdiff


@dataclass
class Instruction:
    """One unit of work for one worker.  Subclasses are dataclasses whose field
    order *is* the device word layout."""

    # opcode -> class, filled by __init_subclass__ for every class that
    # defines a concrete opcode; lets from_words decode a queue.
    _REGISTRY: ClassVar[dict[int, type]] = {}

    def __init_subclass__(cls, **kwargs):
        super().__init_subclass__(**kwargs)
        try:
            code = cls.opcode()
        except NotImplementedError:
            return
        Instruction._REGISTRY[code] = cls

    @classmethod
    def opcode(cls) -> int:
        raise NotImplementedError

    @classmethod
    def prev_opcode(cls) -> int:
        raise NotImplementedError

    @classmethod
    def tags(cls) -> dict[str, Any]:
        return {}

    def cost(self, globs: BaseGlobals) -> float:
        return 0

    def serialize(self) -> list[int]:
        """Word encoding, reference ``instructions.py:97-119``."""
        words: list[int] = [self.opcode()]
        for f in fields(self):
            if f.name == "global_idx":
                continue
            value = getattr(self, f.name)
            if value is None:
                words.append(0)
            elif isinstance(value, (bool, int)):
                words.append(int(value))
            elif isinstance(value, (list, tuple)):
                words.append(len(value))
                words.extend(int(v) for v in value)
            else:
                raise ValueError(f"Unsupported field type: {value!r}")
        return words

    @staticmethod
    def from_words(words) -> "Instruction":
        """Inverse of :meth:`serialize` for a (possibly zero-padded) word row.
        A trailing ``Optional[int]`` field decodes to its integer value, since
        the encoding does not distinguish ``None`` from 0."""
        words = [int(w) for w in words]
        cls = Instruction._REGISTRY.get(words[0])
        if cls is None:
            raise ValueError(f"unknown opcode {words[0]}")
        hints = typing.get_type_hints(cls)
        cursor = 1
        kwargs = {}
        for f in fields(cls):
            hint = hints[f.name]
            origin = typing.get_origin(hint)
            if origin in (list, tuple):
                n = words[cursor]
                items = words[cursor + 1 : cursor + 1 + n]
                kwargs[f.name] = list(items) if origin is list else tuple(items)
                cursor += 1 + n
            elif hint is bool:
                kwargs[f.name] = bool(words[cursor])
                cursor += 1
            else:
                kwargs[f.name] = words[cursor]
                cursor += 1
        return cls(**kwargs)


@dataclass
class NoOp(Instruction):
    """Opcode 0: does nothing; queues are padded with it so that every worker
    has the same number of instruction slots (reference ``instructions.py:122-126``,
    ``scheduler.py:287-289``)."""

    @classmethod
    def opcode(cls) -> int:
        return 0

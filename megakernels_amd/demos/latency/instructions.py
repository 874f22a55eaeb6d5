"""The seven opcodes of the low-latency (batch-1 decode) instruction set and
the buffer bundle they operate on.

Field names, field order (= device word order) and opcode numbers follow
reference ``megakernels/demos/latency/instructions.py:9-196``.  Word layouts
as the device interpreter reads them::

    op1  [1, layer, start_block, end_block]              RMSNorm + QKV matvec + RoPE + KV append
    op2  [2, layer, kv_head, num_partials, partial_idx]  attention over one slice of the KV cache
    op3  [3, layer, head_start, num_partials, is_terminal, n, list[n]..., out_idx]
    op4  [4, layer, start_block, end_block, reduction_block]   O projection + residual
    op5  [5, layer, n, block_idx[n]...]                  RMSNorm + up/gate matvec + SiLU
    op6  [6, layer, start_block, end_block, reduction_block]   down projection + residual
    op7  [7, start_block, end_block]                     final RMSNorm + LM head

The reference hard-codes Llama-3.2-1B numbers for the barrier targets
(``latency/python_vm.py:110,132,176,255,283-290``); :class:`Globals` derives them from
the shapes instead, which reproduces 512 / 128 / 4 for the 1B model and extends
to the 8B shapes.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from torch import Tensor

from megakernels_amd.instructions import BaseGlobals, Instruction
from megakernels_amd.utils import assert_div


@dataclass
class Globals(BaseGlobals):
    # activation buffers
    post_ln_rope_q: Tensor
    attn_out: Tensor
    attn_lse_intermediates: Tensor
    attn_out_intermediates: Tensor
    silu_out: Tensor
    logits: Tensor

    skip_attn_reduction: bool

    # block size constants
    up_gate_proj_block_size: int
    down_proj_block_size: int
    o_proj_block_size: int
    lm_head_block_size: int
    matvec_reduction_size: int
    qkv_block_size: int
    attn_kv_block_size: int
    attn_reduction_size: int

    # ---- derived quantities (generalised barrier arithmetic) -------------

    def gqa_ratio(self) -> int:
        return assert_div(self.num_attention_heads, self.num_kv_heads)

    def qkv_blocks_per_head(self) -> int:
        """QKV output blocks that make up one head; op1 bumps
        ``barriers[l, 0, block // this]`` (4 for head_dim 64)."""
        return assert_div(self.head_dim, self.qkv_block_size)

    def o_proj_col_groups(self) -> int:
        """Column groups of width ``matvec_reduction_size`` in an O-projection
        row (1 for the 1B model)."""
        return assert_div(self.hidden_size, self.matvec_reduction_size)

    def down_proj_col_groups(self) -> int:
        """Column groups of width ``matvec_reduction_size`` in a down-projection
        row (4 for the 1B model, 7 for the 8B model)."""
        return assert_div(self.intermediate_size, self.matvec_reduction_size)

    def o_proj_total_jobs(self) -> int:
        """Value ``barriers[l, 3, 0]`` reaches when every O-projection job of a
        layer is done (128 for the 1B model)."""
        return self.o_proj_col_groups() * assert_div(
            self.hidden_size, self.o_proj_block_size
        )

    def up_gate_total_blocks(self) -> int:
        """Value ``barriers[l, 4, 0]`` reaches after op5 (512 for the 1B model)."""
        return assert_div(self.intermediate_size, self.up_gate_proj_block_size)

    def down_proj_total_jobs(self) -> int:
        """Value ``barriers[l, 5, 0]`` reaches after op6 (512 for the 1B model)."""
        return self.down_proj_col_groups() * assert_div(
            self.hidden_size, self.down_proj_block_size
        )


@dataclass
class LayerNorm_QKV_MatVecRopeAppend(Instruction):
    """RMSNorm, QKV matvec for output blocks ``[start, end)``, RoPE on the Q and
    K blocks, Q to ``post_ln_rope_q``, K/V appended to the cache at ``pos_id``."""

    layer_idx: int
    start_output_block_idx: int
    end_output_block_idx: int

    @classmethod
    def opcode(cls) -> int:
        return 1

    @classmethod
    def prev_opcode(cls) -> int:
        return DownProjResidual.opcode()

    def block_indices(self) -> list[int]:
        return list(range(self.start_output_block_idx, self.end_output_block_idx))

    def cost(self, globs: Globals):
        n_blocks = self.end_output_block_idx - self.start_output_block_idx
        return n_blocks * globs.qkv_block_size * globs.hidden_size


@dataclass
class PartialAttention(Instruction):
    """Attention of the ``gqa_ratio`` query heads sharing ``kv_head_idx`` over
    partition ``partial_idx`` of ``num_partials`` of the cached sequence."""

    layer_idx: int
    kv_head_idx: int
    num_partials: int
    partial_idx: int

    @classmethod
    def opcode(cls) -> int:
        return 2

    @classmethod
    def prev_opcode(cls) -> int:
        return LayerNorm_QKV_MatVecRopeAppend.opcode()

    def cost(self, globs: Globals):
        seq_len = globs.pos_id + 1
        # elements of K and V this partition streams
        return (seq_len / self.num_partials) * globs.head_dim * 2


@dataclass
class AttentionReduction(Instruction):
    """Log-sum-exp merge of the partial attention results listed in
    ``reduction_list`` for ``attn_reduction_size`` heads from ``head_start_idx``."""

    layer_idx: int
    head_start_idx: int
    # how many partitions the attention of this layer was split into
    num_partials: int
    is_terminal: bool
    reduction_list: list[int]
    # slot to write a non-terminal merge into (unused for the terminal one)
    output_partial_idx: Optional[int] = None

    @classmethod
    def opcode(cls) -> int:
        return 3

    @classmethod
    def prev_opcode(cls) -> int:
        return PartialAttention.opcode()

    def cost(self, globs: Globals):
        return len(self.reduction_list) * globs.attn_reduction_size * globs.head_dim


@dataclass
class MatVecAdd(Instruction):
    """``residual[rows] += W[rows, group] @ vec[group]`` for output blocks
    ``[start, end)`` and one column group."""

    layer_idx: int
    start_block_idx: int
    end_block_idx: int
    reduction_block_idx: int


@dataclass
class O_ProjResidual(MatVecAdd):
    @classmethod
    def opcode(cls) -> int:
        return 4

    @classmethod
    def prev_opcode(cls) -> int:
        return AttentionReduction.opcode()

    def cost(self, globs: Globals):
        n_blocks = self.end_block_idx - self.start_block_idx
        return n_blocks * globs.o_proj_block_size * globs.matvec_reduction_size


@dataclass
class LayerNormDoubleMatVecSiLU(Instruction):
    """RMSNorm, up and gate matvecs for the listed output blocks,
    ``silu(gate) * up`` to ``silu_out``."""

    layer_idx: int
    block_idxs: list[int]

    @classmethod
    def opcode(cls) -> int:
        return 5

    @classmethod
    def prev_opcode(cls) -> int:
        return O_ProjResidual.opcode()

    def cost(self, globs: Globals):
        # two matrices per block
        return len(self.block_idxs) * globs.up_gate_proj_block_size * globs.hidden_size * 2


@dataclass
class DownProjResidual(MatVecAdd):
    @classmethod
    def opcode(cls) -> int:
        return 6

    @classmethod
    def prev_opcode(cls) -> int:
        return LayerNormDoubleMatVecSiLU.opcode()

    def cost(self, globs: Globals):
        n_blocks = self.end_block_idx - self.start_block_idx
        return n_blocks * globs.down_proj_block_size * globs.matvec_reduction_size


@dataclass
class RMS_LM_Head(Instruction):
    """Final RMSNorm and LM-head matvec for logit blocks ``[start, end)``."""

    start_output_block_idx: int
    end_output_block_idx: int

    @classmethod
    def opcode(cls) -> int:
        return 7

    @classmethod
    def prev_opcode(cls) -> int:
        return DownProjResidual.opcode()

    def cost(self, globs: Globals):
        n_blocks = self.end_output_block_idx - self.start_output_block_idx
        return n_blocks * globs.lm_head_block_size * globs.hidden_size

"""TEST INFRASTRUCTURE: a second, independent restatement of the reference's
Python VM, written with the same torch operations the reference uses
(``megakernels/demos/latency/python_vm.py``), so that the only difference to
the reference is the author.  It exists to pin the C checker: the C checker
fixes a summation order of its own, so the two agree within bf16 rounding, not
bit for bit (the tests state the tolerance).

Differences to the reference, all of them generalisations that reproduce the
reference's numbers for Llama-3.2-1B: barrier targets are derived from the
shapes (512 / 128 / 4 in ``python_vm.py:110,132,176,255,283-290``), and the O
projection accepts any column group (``:88-89`` asserts group 0).
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F

from megakernels_amd.demos.latency.instructions import (
    AttentionReduction,
    DownProjResidual,
    Globals,
    LayerNorm_QKV_MatVecRopeAppend,
    LayerNormDoubleMatVecSiLU,
    O_ProjResidual,
    PartialAttention,
    RMS_LM_Head,
)
from megakernels_amd.instructions import NoOp

BLOCK = 16


def _expect(globs: Globals, layer: int, row: int, col: int, want: int):
    have = int(globs.barriers[layer, row, col])
    assert have == want, f"barriers[{layer},{row},{col}] is {have}, expected {want}"


def _rms(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    x32 = x.float()
    scale = torch.rsqrt(x32.square().mean(-1, keepdim=True) + eps)
    return w * (x32 * scale).to(x.dtype)


def _rope_pairs(vec: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Interleaved rotary embedding on a slice whose first element sits at an
    even head-dimension index; bf16 in, fp32 out (the bf16 * fp32 product
    promotes to fp32, ``llama.py:170-173``)."""
    pairs = vec.view(-1, 2)
    rotated = torch.stack((-pairs[:, 1], pairs[:, 0]), dim=-1).reshape(-1)
    return vec * cos + rotated * sin


def qkv_rope_append(g: Globals, ins: LayerNorm_QKV_MatVecRopeAppend):
    layer = ins.layer_idx
    if layer > 0:
        _expect(g, layer - 1, 5, 0, g.down_proj_total_jobs())
    x = _rms(g.hidden_states, g.attn_ln_weights[layer], g.rms_norm_eps)
    D = g.head_dim
    k0 = g.num_attention_heads * D
    v0 = k0 + g.num_kv_heads * D
    pos = g.pos_id
    for b in range(ins.start_output_block_idx, ins.end_output_block_idx):
        lo, hi = b * BLOCK, (b + 1) * BLOCK
        y = torch.mv(g.qkv_proj_weights[layer][lo:hi], x)
        if lo < v0:
            d = lo % D
            y = _rope_pairs(y, g.rope_cos[pos, d : d + BLOCK], g.rope_sin[pos, d : d + BLOCK])
        if lo < k0:
            g.post_ln_rope_q[lo:hi] = y
        elif lo < v0:
            g.k_cache[layer, 0, pos].view(-1)[lo - k0 : hi - k0] = y
        else:
            g.v_cache[layer, 0, pos].view(-1)[lo - v0 : hi - v0] = y
        g.barriers[layer, 0, b // g.qkv_blocks_per_head()] += 1


def partial_attention(g: Globals, ins: PartialAttention):
    layer, kvh = ins.layer_idx, ins.kv_head_idx
    gqa = g.gqa_ratio()
    H, KVH = g.num_attention_heads, g.num_kv_heads
    per_head = g.qkv_blocks_per_head()
    for col in [*range(kvh * gqa, (kvh + 1) * gqa), H + kvh, H + KVH + kvh]:
        _expect(g, layer, 0, col, per_head)

    seq_len = g.pos_id + 1
    total_blocks = math.ceil(seq_len / g.attn_kv_block_size)
    per_partial = math.ceil(total_blocks / ins.num_partials)
    first = ins.partial_idx * per_partial
    last = min(first + per_partial, total_blocks)
    t0 = first * g.attn_kv_block_size
    t1 = min(last * g.attn_kv_block_size, seq_len)

    k = g.k_cache[layer, 0, t0:t1, kvh].float()
    v = g.v_cache[layer, 0, t0:t1, kvh].float()
    heads = slice(kvh * gqa, (kvh + 1) * gqa)
    q = g.post_ln_rope_q.view(H, -1)[heads].float()

    scores = (q @ k.T) * g.attn_scale
    probs = torch.softmax(scores, dim=-1)
    lse = torch.log2(torch.exp(scores).sum(dim=-1))
    out = probs @ v

    if g.skip_attn_reduction:
        g.attn_out.view(H, -1)[heads] = out
        g.barriers[layer, 2, 0] += gqa
    else:
        g.attn_lse_intermediates[heads, ins.partial_idx] = lse
        g.attn_out_intermediates[heads, ins.partial_idx] = out
        g.barriers[layer, 1, heads] += 1


def attention_reduction(g: Globals, ins: AttentionReduction):
    layer, h0 = ins.layer_idx, ins.head_start_idx
    # the reference asserts equality (python_vm.py:354); in a reduction tree, which it never schedules,
    # the counter also holds the finished merges below this one
    have = int(g.barriers[layer, 1, h0])
    assert have >= ins.num_partials, f"barriers[{layer},1,{h0}] is {have}, expected at least {ins.num_partials}"
    heads = slice(h0, h0 + g.attn_reduction_size)
    idx = torch.tensor(ins.reduction_list, dtype=torch.long)
    lses = g.attn_lse_intermediates[heads][:, idx]
    outs = g.attn_out_intermediates[heads][:, idx]
    top = lses.max(dim=-1, keepdim=True).values
    # all listed partitions empty (possible for a run of a reduction tree past the end of the
    # sequence): the formula gives NaN; the merge of nothing is nothing, zeros and lse -inf
    nothing = torch.isneginf(top)
    weights = torch.where(nothing, torch.zeros_like(lses), (lses - top).exp2())
    denom = weights.sum(dim=-1, keepdim=True)
    merged = torch.where(nothing, torch.zeros_like(outs[:, 0]), (outs * weights.unsqueeze(-1)).sum(dim=1) / denom)
    if ins.is_terminal:
        g.attn_out.view(g.num_attention_heads, -1)[heads] = merged
    else:
        new_lse = torch.where(nothing, top, top + denom.log2())
        g.attn_lse_intermediates[heads, ins.output_partial_idx] = new_lse.squeeze(-1)
        g.attn_out_intermediates[heads, ins.output_partial_idx] = merged
    # the reference bumps row 2 after every reduction (python_vm.py:391-392), which would open the O
    # projection's barrier before a tree is done: a non-terminal merge counts as one more partial
    # result of its heads instead
    if ins.is_terminal:
        g.barriers[layer, 2, 0] += g.attn_reduction_size
    else:
        g.barriers[layer, 1, heads] += 1


def _matvec_residual(mat, vec, residual, ins, R):
    cols = slice(ins.reduction_block_idx * R, (ins.reduction_block_idx + 1) * R)
    for b in range(ins.start_block_idx, ins.end_block_idx):
        rows = slice(b * BLOCK, (b + 1) * BLOCK)
        residual[rows] += torch.mv(mat[rows, cols], vec[cols])


def o_proj_residual(g: Globals, ins: O_ProjResidual):
    _expect(g, ins.layer_idx, 2, 0, g.num_attention_heads)
    _matvec_residual(g.o_proj_weights[ins.layer_idx], g.attn_out, g.hidden_states, ins, g.matvec_reduction_size)
    g.barriers[ins.layer_idx, 3, 0] += ins.end_block_idx - ins.start_block_idx


def down_proj_residual(g: Globals, ins: DownProjResidual):
    _expect(g, ins.layer_idx, 4, 0, g.up_gate_total_blocks())
    _matvec_residual(g.down_proj_weights[ins.layer_idx], g.silu_out, g.hidden_states, ins, g.matvec_reduction_size)
    g.barriers[ins.layer_idx, 5, 0] += ins.end_block_idx - ins.start_block_idx


def upgate_silu(g: Globals, ins: LayerNormDoubleMatVecSiLU):
    layer = ins.layer_idx
    _expect(g, layer, 3, 0, g.o_proj_total_jobs())
    x = _rms(g.hidden_states, g.mlp_ln_weights[layer], g.rms_norm_eps)
    for b in ins.block_idxs:
        rows = slice(b * BLOCK, (b + 1) * BLOCK)
        up = torch.mv(g.up_proj_weights[layer][rows], x)
        gate = torch.mv(g.gate_proj_weights[layer][rows], x)
        g.silu_out[rows] = F.silu(gate) * up
        g.barriers[layer, 4, 0] += 1


def rms_lm_head(g: Globals, ins: RMS_LM_Head):
    _expect(g, g.num_hidden_layers - 1, 5, 0, g.down_proj_total_jobs())
    x = _rms(g.hidden_states, g.lm_head_norm_weights, g.rms_norm_eps)
    for b in range(ins.start_output_block_idx, ins.end_output_block_idx):
        rows = slice(b * BLOCK, (b + 1) * BLOCK)
        g.logits[rows] = torch.mv(g.lm_head_weights[rows], x)


SOLVERS = {
    NoOp: lambda g, ins: None,
    LayerNorm_QKV_MatVecRopeAppend: qkv_rope_append,
    PartialAttention: partial_attention,
    AttentionReduction: attention_reduction,
    O_ProjResidual: o_proj_residual,
    LayerNormDoubleMatVecSiLU: upgate_silu,
    DownProjResidual: down_proj_residual,
    RMS_LM_Head: rms_lm_head,
}


@torch.inference_mode()
def interpret(globs: Globals, instructions) -> None:
    for ins in instructions:
        SOLVERS[type(ins)](globs, ins)

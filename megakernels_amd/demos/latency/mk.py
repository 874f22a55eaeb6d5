"""Argument marshalling for one megakernel launch.

The positional order is the boundary contract of reference
``megakernels/demos/latency/mk.py:15-49`` (and of the binding it calls,
``demos/low-latency-llama/llama.cu:28-52``): barriers, instructions, timings,
nine weight tensors, K and V caches viewed as ``[(L B), T, KVH, D]``, the two
rope tables, seven activation buffers, then ``pos_id``, ``attn_scale``,
``rms_norm_eps``, ``skip_attn_reduction`` and the keyword ``stream``.
"""

from __future__ import annotations

import torch

from megakernels_amd.demos.latency.instructions import Globals
from megakernels_amd.mk import MK_Interpreter


def interpret_with_mk(globs: Globals, mk_func, **fused):
    # [L, B, T, KVH, D] -> [(L B), T, KVH, D]; a view, the cache is contiguous
    k_cache_4d = globs.k_cache.flatten(0, 1)
    v_cache_4d = globs.v_cache.flatten(0, 1)

    mk_func(
        # vm state
        globs.barriers,
        globs.instructions,
        globs.timings,
        # weights
        globs.qkv_proj_weights,
        globs.attn_ln_weights,
        globs.o_proj_weights,
        globs.mlp_ln_weights,
        globs.up_proj_weights,
        globs.gate_proj_weights,
        globs.down_proj_weights,
        globs.lm_head_norm_weights.data,
        globs.lm_head_weights.data,
        k_cache_4d,
        v_cache_4d,
        # rope
        globs.rope_cos,
        globs.rope_sin,
        # activations
        globs.hidden_states,
        globs.post_ln_rope_q,
        globs.attn_out,
        globs.attn_lse_intermediates,
        globs.attn_out_intermediates,
        globs.silu_out,
        globs.logits,
        # scalars
        globs.pos_id,
        globs.attn_scale,
        globs.rms_norm_eps,
        globs.skip_attn_reduction,
        stream=torch.cuda.current_stream(),
        **fused,
    )


class LatencyMK_Interpreter(MK_Interpreter):
    def interpret(self, globs: Globals):
        interpret_with_mk(globs, self.mk_func)

    def interpret_step(self, globs: Globals, embed_table, token_in, token_out):
        """One whole decode step in one launch: embedding row of ``token_in``,
        the instruction stream, ``argmax`` into ``token_out``, barriers left
        zeroed (no counterpart in the reference, whose loop does these around
        the launch, ``megakernels/generators.py:121-143``)."""
        interpret_with_mk(globs, self.mk_func, embed_table=embed_table, token_in=token_in,
                          token_out=token_out, reset_barriers=True)

    def interpret_steps(self, globs: Globals, embed_table, token_in, tokens_out):
        """``len(tokens_out)`` decode steps in one launch, starting at
        ``globs.pos_id``: step ``s`` consumes the token of step ``s - 1``
        (``token_in`` for the first) and writes ``tokens_out[s]``.  The
        reference launches once per token (``megakernels/generators.py:121-143``)."""
        interpret_with_mk(globs, self.mk_func, embed_table=embed_table, token_in=token_in,
                          token_out=tokens_out, reset_barriers=True, num_steps=tokens_out.numel())

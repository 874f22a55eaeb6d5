"""Writes tests/golden/reference_schedules.json from the reference's own scheduler.

Run in the development container only (the reference tree does not travel):

    python tests/golden/make_schedule_fixtures.py /root/reference

It imports the reference's pure-integer scheduling code
(megakernels/demos/latency/scheduler.py, megakernels/scheduler.py,
megakernels/instructions.py) with the worker count patched to a fixed number
(the reference reads it from a CUDA device) and a buffer bundle that holds no
tensors, builds the Llama-3.2-1B schedule for 132 and 148 workers, and stores
the serialized instruction words: the linear order for layers 0-1 plus LM head,
and the per-worker queues of every assignment policy.  These are the parts of
the schedule that only a run of the reference can pin against transcription
slips (the down-projection run splitting, Python's round-half-even block
boundaries, the heap order of the DAG assignment).
"""

import json
import sys
from pathlib import Path


def main(reference_root: str):
    sys.path.insert(0, reference_root)
    import megakernels.utils as ref_utils

    workers_box = {"n": 132}
    ref_utils.get_sm_count = lambda device=None: workers_box["n"]
    import megakernels.instructions as ref_instructions

    ref_instructions.get_sm_count = ref_utils.get_sm_count
    import megakernels.demos.latency.scheduler as ref_latency
    import megakernels.scheduler as ref_sched
    from megakernels.demos.latency.instructions import Globals

    ref_latency.get_sm_count = ref_utils.get_sm_count

    def make_globs():
        return Globals(
            qkv_proj_weights=None, attn_ln_weights=None, o_proj_weights=None, mlp_ln_weights=None,
            up_proj_weights=None, gate_proj_weights=None, down_proj_weights=None,
            lm_head_norm_weights=None, lm_head_weights=None, k_cache=None, v_cache=None,
            rope_cos=None, rope_sin=None,
            num_hidden_layers=2, num_attention_heads=32, num_kv_heads=8, head_dim=64,
            hidden_size=2048, intermediate_size=8192, vocab_size=128256,
            attn_scale=0.125, rms_norm_eps=1e-5, device="cpu",
            hidden_states=None, barriers=None, pos_id=40,
            post_ln_rope_q=None, attn_out=None, attn_lse_intermediates=None,
            attn_out_intermediates=None, silu_out=None, logits=None,
            skip_attn_reduction=True,
            up_gate_proj_block_size=16, down_proj_block_size=16, o_proj_block_size=16,
            lm_head_block_size=16, matvec_reduction_size=2048, qkv_block_size=16,
            attn_kv_block_size=16, attn_reduction_size=4,
        )

    out = {}
    for workers in (132, 148):
        workers_box["n"] = workers
        globs = make_globs()
        nodes, end_node = ref_latency.make_dag(globs)
        schedule = ref_sched.Schedule(globs, nodes, end_node)
        linear = [ins.serialize() for ins in schedule.get_linear_instructions()]
        entry = {"linear": linear, "queues": {}}
        for mode in ("rr", "zz", "wave", "dag"):
            nodes, end_node = ref_latency.make_dag(make_globs())
            sched = ref_sched.Schedule(globs, nodes, end_node)
            queues = ref_sched.assign_to_sms(mode, schedule=sched)
            entry["queues"][mode] = [[ins.serialize() for ins in q] for q in queues]
        out[str(workers)] = entry
    target = Path(__file__).parent / "reference_schedules.json"
    target.write_text(json.dumps(out, separators=(",", ":")))
    print("wrote", target, target.stat().st_size, "bytes")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")

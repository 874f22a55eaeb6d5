"""Manual bisection harness, counterpart of the reference's ``scripts/diff_test.py``: run the CPU
checker and the HIP megakernel on the same random hidden state / KV cache (valid positions N(0,1),
positions beyond the sequence N(0,100) as poison) and print, per buffer, the largest absolute
difference, the mean relative difference and the number of differing elements.  Needs a GPU.

    python tests/diff_test.py model=1b layer_limit=1 stop_after_op=oproj prompt_len=10 ntok=10
    python tests/diff_test.py model=tiny .full num_attention_partitions=3
    python tests/diff_test.py model=1b layer_limit=1 start_after_op=oproj

``start_after_op`` (reference ``diff_test.py:122-152,198-208``): the checker runs the instructions up to and
including that op on both sets of buffers, the megakernel gets only the rest.

It lives with the tests because it drives the checker, which the product never imports.
"""

from __future__ import annotations

import sys
from dataclasses import dataclass, fields
from pathlib import Path

import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
sys.path.insert(0, str(Path(__file__).resolve().parent))

from helpers import build_schedule, config_8b_slice, config_tiny, fill_kv, make_model, mirror_to_gpu, mismatches  # noqa: E402
from megakernels_amd.llama import LlamaConfig  # noqa: E402


@dataclass
class ScriptConfig:
    model: str = "1b"
    prompt_len: int = 10
    ntok: int = 10
    stop_after_op: str | None = None
    start_after_op: str | None = None
    layer_limit: int | None = 1
    sched: str = "rr"
    workers: int = 256
    num_attention_partitions: int = 1
    barrier_init_val: int = 0
    noops: bool = False
    outfile: str | None = None

    def full(self):
        self.layer_limit = None


def parse(argv):
    cfg = ScriptConfig()
    for arg in argv:
        if arg.startswith("."):
            getattr(cfg, arg[1:])()
            continue
        key, _, value = arg.partition("=")
        current = getattr(cfg, key)
        if value in ("None", "none"):
            setattr(cfg, key, None)
        elif isinstance(current, bool):
            setattr(cfg, key, value.lower() in ("1", "true"))
        elif key == "outfile":
            setattr(cfg, key, value)
        elif isinstance(current, int) or key in ("layer_limit",):
            setattr(cfg, key, int(value))
        else:
            setattr(cfg, key, value)
    return cfg


def main(config: ScriptConfig):
    from megakernels_amd.demos.latency.mk import LatencyMK_Interpreter
    from oracle import pyvm

    arch = {"1b": LlamaConfig.llama_1b(), "8b": LlamaConfig.llama_8b(), "tiny": config_tiny(),
            "8b_slice": config_8b_slice()}[config.model]
    if config.layer_limit is not None and config.model in ("1b", "8b"):
        # building all layers' weights to run one is wasteful: keep two
        arch.num_hidden_layers = max(2, config.layer_limit)
    if config.model == "tiny":
        config.workers = 16
    seq_len = config.prompt_len + config.ntok
    model = make_model(arch, max_len=max(256, seq_len + 16))
    fill_kv(model, upto=seq_len)
    schedule = build_schedule(model, config.workers, partitions=config.num_attention_partitions,
                              sched=config.sched, stop_after_op=config.stop_after_op, layer_limit=config.layer_limit)
    g = schedule.globs
    g.hidden_states.normal_()
    g.pos_id = seq_len - 1
    g.barriers.fill_(config.barrier_init_val)
    instructions = schedule.get_linear_instructions()
    if config.start_after_op is not None:
        from megakernels_amd.scheduler import assign_to_sms, tensorize_instructions

        head = build_schedule(model, config.workers, partitions=config.num_attention_partitions, sched=config.sched,
                              stop_after_op=config.start_after_op, layer_limit=config.layer_limit).get_linear_instructions()
        assert len(head) < len(instructions) and instructions[: len(head)] == head, "start_after_op must come before the end"
        print(f"running the first {len(head)} of {len(instructions)} instructions with the checker...")
        pyvm.interpret(g, head, check_barriers=config.barrier_init_val == 0)
        instructions = instructions[len(head):]
        tensorize_instructions(g, assign_to_sms("rr", instructions=instructions, sm_count=config.workers))
    if config.noops:
        g.instructions.zero_()
    queue_lengths = [int((q[:, 0] != 0).sum()) for q in g.instructions]
    print(f"worker queue lengths: min={min(queue_lengths)}, max={max(queue_lengths)}, "
          f"mean={sum(queue_lengths) / len(queue_lengths):.2f}")
    _, schedule_gpu = mirror_to_gpu(model, schedule)
    if config.noops:
        instructions = []
    pyvm.interpret(g, instructions, check_barriers=config.barrier_init_val == 0)
    interp = LatencyMK_Interpreter()
    mk_mod = sys.modules["mk_llama"]
    mk_mod.record_timings = config.outfile is not None
    try:
        interp.interpret(schedule_gpu.globs)
        mk_mod.check_status("cuda:0")
    finally:
        mk_mod.record_timings = False
    print("done! diffing tensors:")
    g.diff(schedule_gpu.globs.__class__(**{f.name: (getattr(schedule_gpu.globs, f.name).cpu()
           if isinstance(getattr(schedule_gpu.globs, f.name), torch.Tensor) else getattr(schedule_gpu.globs, f.name))
           for f in fields(schedule_gpu.globs)}))
    print("elements that differ bit for bit:", mismatches(g, schedule_gpu.globs) or "none")
    if config.outfile is not None:
        # the reference's dump (scripts/diff_test.py:231-242): timings, instruction words, the
        # instruction objects per worker and the summed cost per worker.  `timings` is in the
        # reference's event slots (include/util.cuh:215-246); `timings_native` as the kernel wrote them.
        import pickle

        from megakernels_amd.scheduler import assign_to_sms
        from megakernels_amd.scripts.timeline import reference_event_layout

        if config.start_after_op is None:
            queues = assign_to_sms(config.sched, schedule=schedule)
        else:
            queues = assign_to_sms("rr", instructions=instructions, sm_count=config.workers)
        gg = schedule_gpu.globs
        outdata = {
            "timings": reference_event_layout(gg.timings, gg.instructions),
            "timings_native": gg.timings.cpu(),
            "instructions": gg.instructions.cpu(),
            "python_instructions": queues,
            "cost_per_sm": [sum(ins.cost(g) for ins in q) for q in queues],
        }
        print(f"Saving to {config.outfile}")
        with open(config.outfile, "wb") as f:
            pickle.dump(outdata, f)


if __name__ == "__main__":
    main(parse(sys.argv[1:]))
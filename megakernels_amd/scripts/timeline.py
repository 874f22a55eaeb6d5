"""Per-instruction timeline of one decode step, from the megakernel's own timing records.

    python -m megakernels_amd.scripts.timeline [model=1b] [layers=16] [pos=4100] [partitions=0] [layer=1]
                                               [sched=rr] [out=trace.npz]

Builds the random-initialised 1B (or ``model=8b``) architecture with ``layers`` layers, fills the KV cache up to ``pos``
with seeded noise, runs a few warm-up steps, then one step with ``MK_FLAG_TIMINGS`` set and prints,
per instruction kind, how long the workers waited for the dependency, loaded the activation vector,
computed and wrote back; and for one layer when each kind started, saw its dependency and ended across
the workers.  ``out=`` saves the raw records (``timings`` [workers, slots, 128] and ``instructions``
[workers, slots, 32], plain ``numpy`` arrays, plus ``reference_layout``: the same records in the
reference's event slots, ``include/util.cuh:215-246``) for a Gantt view elsewhere; the dump shaped like the
reference's ``diff_test.py outfile=`` (``scripts/diff_test.py:231-242``) comes from ``tests/diff_test.py outfile=``.  The reference records the
same events (``include/util.cuh:215-246``) when compiled with ``TIMING_RECORD_ENABLED``; here the records
are taken on request at run time.

Times are microseconds since the first workgroup took its first instruction (100 MHz wall clock of the
device, common to all compute units).
"""

from __future__ import annotations

import sys

import numpy as np
import torch

from megakernels_amd.demos.latency.scheduler import LatencyScheduleBuilder, pick_num_attention_partitions
from megakernels_amd.dispatch import make_mk_interpreter
from megakernels_amd.llama import LlamaConfig, LlamaForCausalLM
from megakernels_amd.model_types import ExtraModelConfig
from megakernels_amd.scheduler import assign_to_sms, tensorize_instructions
from megakernels_amd.utils import get_sm_count, set_sm_count_override

NAMES = {1: "qkv", 2: "attention", 3: "merge", 4: "o-proj", 5: "up/gate", 6: "down", 7: "lm-head"}

# The reference's event slots (include/util.cuh:215-246) and the record of this kernel (MK_TIMING_* of
# include/mk_llama.h: 0 start, 1 dependency seen, 2 input ready, 3 rows done, 4 end) each one is taken
# from.  The reference's stages that this kernel does not have (instruction fetch, page allocation,
# semaphore set-up: all done before an instruction starts here) get the start time.
REFERENCE_EVENTS = {
    0: 0,    # TEVENT_CONTROLLER_START
    1: 0,    # TEVENT_IFETCH_DONE
    2: 0,    # TEVENT_PAGE_ALLOC_DONE
    3: 0,    # TEVENT_SEMS_SETUP
    4: 4,    # TEVENT_CONTROLLER_END
    5: 0,    # TEVENT_LOADER_START: the first weight rows are requested on entry
    7: 2,    # TEVENT_LAUNCHER_START
    9: 3,    # TEVENT_STORER_START
    11: 2,   # TEVENT_CONSUMER_START
    44: 0,   # TEVENT_AT_GMEM_WAIT
    45: 1,   # TEVENT_DONE_GMEM_WAIT
    46: 3,   # TEVENT_AT_GMEM_STORE
    47: 4,   # TEVENT_DONE_GMEM_STORE
    48: 0,   # TEVENT_FIRST_LOAD
    49: 2,   # TEVENT_FIRST_USE
    50: 3,   # TEVENT_FIRST_STORE
    51: 3,   # TEVENT_LAST_LOAD
    52: 3,   # TEVENT_LAST_USE
    53: 4,   # TEVENT_LAST_STORE
    54: 4,   # TEVENT_OUTPUT_READY
}


def launch_origin(starts) -> int:
    """The earliest of the 32-bit clock values ``starts`` (a 1-D integer tensor or array), when they lie
    within half the clock's range of each other - also if the clock wrapped in between."""
    v = np.asarray(starts).astype(np.int64) & 0xFFFFFFFF
    first = int(v[0])
    signed = ((v - first + (1 << 31)) % (1 << 32)) - (1 << 31)
    return (first + int(signed.min())) % (1 << 32)


def reference_event_layout(timings: torch.Tensor, instructions: torch.Tensor) -> torch.Tensor:
    """``timings [workers, slots, 128]`` of this kernel re-laid as the reference's tools expect them:
    the slots of ``REFERENCE_EVENTS`` filled, as ticks (10 ns) since the first instruction of the
    launch started; everything else zero, as are the rows of NoOp padding."""
    t = timings.cpu().to(torch.int64)
    ins = instructions.cpu()
    executed = ins[:, :, 0] != 0
    out = torch.zeros_like(t)
    if not bool(executed.any()):
        return out.to(torch.int32)
    origin = launch_origin(t[:, :, 0][executed].numpy())
    ticks = ((t[:, :, :5] & 0xFFFFFFFF) - origin) % (1 << 32)
    for slot, source in REFERENCE_EVENTS.items():
        out[:, :, slot] = torch.where(executed, ticks[:, :, source], torch.zeros_like(ticks[:, :, source]))
    return out.to(torch.int32)


def main(argv):
    opts = {"model": "1b", "layers": 16, "pos": 4100, "partitions": 0, "layer": 1, "sched": "rr", "out": ""}
    for arg in argv:
        key, _, value = arg.partition("=")
        if key not in opts:
            raise SystemExit(f"unknown option {key}; known: {', '.join(opts)}")
        opts[key] = value if key in ("model", "sched", "out") else int(value)
    if not torch.cuda.is_available():
        raise SystemExit("timeline needs a GPU")
    device = torch.device("cuda:0")
    if opts["model"] not in ("1b", "8b"):
        raise SystemExit("model is 1b or 8b")
    cfg = LlamaConfig.llama_1b() if opts["model"] == "1b" else LlamaConfig.llama_8b()
    cfg.num_hidden_layers = opts["layers"]
    pos = opts["pos"]
    model = LlamaForCausalLM.from_random(cfg, ExtraModelConfig(interleave_rope=True, max_len_override=pos + 64), seed=0)
    gen = torch.Generator().manual_seed(2)
    for cache in model.stacked_kv_cache:
        shape = list(cache.shape)
        shape[2] = pos
        cache[:, :, :pos] = torch.randn(shape, generator=gen).to(cache.dtype)
    model = model.to(device)
    workers = get_sm_count(device)
    set_sm_count_override(workers)
    partitions = opts["partitions"] or pick_num_attention_partitions(pos, 1, device, cfg.num_key_value_heads, cfg.head_dim)
    schedule = LatencyScheduleBuilder.build(model, num_attention_partitions=partitions)
    tensorize_instructions(schedule.globs, assign_to_sms(opts["sched"], schedule=schedule))
    globs = schedule.globs
    interpreter = make_mk_interpreter("latency")
    mk = sys.modules["mk_llama"]
    globs.hidden_states.copy_(model.model.embed_tokens.weight[5])
    globs.pos_id = pos
    for _ in range(3):
        globs.barriers.zero_()
        interpreter.interpret(globs)
    mk.check_status(device)
    mk.record_timings = True
    globs.barriers.zero_()
    globs.timings.zero_()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    interpreter.interpret(globs)
    end.record()
    torch.cuda.synchronize()
    mk.record_timings = False
    mk.check_status(device)

    # [workers, slots, 6]: start, dependency seen, activation ready, rows done, end, opcode
    t = globs.timings.cpu()[:, :, :6].numpy().astype(np.float64)
    ins = globs.instructions.cpu().numpy()
    # the records are the low 32 bits of the device clock: times since the earliest record
    executed = t[:, :, 5] != 0
    origin = np.int64(launch_origin(globs.timings.cpu()[:, :, 0].numpy()[executed]))
    t[:, :, :5] = ((t[:, :, :5].astype(np.int64) - origin) % (1 << 32)) / 100.0
    if opts["out"]:
        np.savez_compressed(opts["out"], timings=globs.timings.cpu().numpy(), instructions=ins,
                            reference_layout=reference_event_layout(globs.timings, globs.instructions).numpy(),
                            ticks_per_microsecond=np.array(100))
    print(f"{opts['model']}, {opts['layers']} layers, position {pos}, {partitions} attention partitions, {workers} workers, "
          f"assignment {opts['sched']}: kernel {start.elapsed_time(end) * 1e3:.1f} us with timing records on, "
          f"last instruction ends at {t[:, :, 4].max():.1f} us")
    print("\nper instruction kind, mean / max over all instructions (us):")
    print(f"{'kind':10s} {'count':>6s} {'wait for dependency':>20s} {'activation':>14s} {'rows':>14s} {'write back':>14s}")
    for op, name in NAMES.items():
        sel = t[:, :, 5] == op
        if not sel.any():
            continue
        st, dep, inp, rows, done = (t[:, :, i][sel] for i in range(5))
        if op in (2, 3):
            inp = dep  # these record no separate activation event
        cell = lambda a: f"{a.mean():6.2f} /{a.max():6.2f}"
        print(f"{name:10s} {int(sel.sum()):6d} {cell(dep - st):>20s} {cell(inp - dep):>14s} {cell(rows - inp):>14s} {cell(done - rows):>14s}")
    layer = min(opts["layer"], opts["layers"] - 1)
    print(f"\nlayer {layer}, over the workers that run the kind (us): first start | dependency seen p10 p50 max | end p10 p50 max")
    for op in range(1, 7):
        sel = (ins[:, :, 0] == op) & (ins[:, :, 1] == layer)
        if not sel.any():
            continue
        st, dep, done = t[:, :, 0][sel], t[:, :, 1][sel], t[:, :, 4][sel]
        q = lambda a, ps: " ".join(f"{np.percentile(a, p):7.2f}" for p in ps)
        print(f"  {NAMES[op]:10s} {st.min():7.2f} | {q(dep, (10, 50, 100))} | {q(done, (10, 50, 100))}")
    sel = ins[:, :, 0] == 7
    if sel.any():
        print(f"  {'lm-head':10s} {t[:, :, 0][sel].min():7.2f} | {np.percentile(t[:, :, 1][sel], 50):7.2f} (p50) | "
              f"{t[:, :, 4][sel].max():7.2f} (max)")


if __name__ == "__main__":
    main(sys.argv[1:])

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

# Slots of a timing record (MK_TIMING_* of include/mk_llama.h; the reference's TEVENT_* of
# include/util.cuh:215-246 where the names agree).
START, DEP_READY, INPUT_READY, COMPUTE_DONE, END = 0, 1, 2, 3, 4
LOADER_START, LAUNCHER_START, STORER_START, CONSUMER_START = 5, 7, 9, 11
AT_GMEM_WAIT, DONE_GMEM_WAIT, AT_GMEM_STORE, DONE_GMEM_STORE = 44, 45, 46, 47
FIRST_LOAD, FIRST_USE, FIRST_STORE, LAST_LOAD, LAST_USE, LAST_STORE, OUTPUT_READY = 48, 49, 50, 51, 52, 53, 54
OPCODE, ATTN_MAXIMA, ATTN_PROBABILITIES = 55, 56, 57
CONSUMER_WAVES = 8
# every slot that holds a time
TIME_SLOTS = ([START, DEP_READY, INPUT_READY, COMPUTE_DONE, END, LOADER_START, LAUNCHER_START, STORER_START]
              + list(range(CONSUMER_START, CONSUMER_START + 2 * CONSUMER_WAVES))
              + list(range(AT_GMEM_WAIT, OUTPUT_READY + 1)) + [ATTN_MAXIMA, ATTN_PROBABILITIES])
# The reference's stages that this kernel does not have (instruction fetch, page allocation, semaphore
# set-up: the queue is in LDS, there are no pages or semaphores) are over when an instruction starts.
REFERENCE_ONLY_STAGES = (1, 2, 3)   # TEVENT_IFETCH_DONE, TEVENT_PAGE_ALLOC_DONE, TEVENT_SEMS_SETUP


def launch_origin(starts) -> int:
    """The earliest of the 32-bit clock values ``starts`` (a 1-D integer tensor or array), when they lie
    within half the clock's range of each other - also if the clock wrapped in between."""
    v = np.asarray(starts).astype(np.int64) & 0xFFFFFFFF
    first = int(v[0])
    signed = ((v - first + (1 << 31)) % (1 << 32)) - (1 << 31)
    return (first + int(signed.min())) % (1 << 32)


def reference_event_layout(timings: torch.Tensor, instructions: torch.Tensor) -> torch.Tensor:
    """``timings [workers, slots, 128]`` as the reference's tools expect them: every event the kernel
    stamped, in the reference's slot, as ticks (10 ns) since the first instruction of the launch
    started; slots 1-3 (stages only the reference has) hold the start; a slot the kernel did not stamp
    for an instruction (a wave without rows, an instruction kind without that stage) is zero, as are
    the rows of NoOp padding.  Slot 55, the reference's first free one, keeps the opcode."""
    t = timings.cpu().to(torch.int64)
    ins = instructions.cpu()
    executed = ins[:, :, 0] != 0
    out = torch.zeros_like(t)
    if not bool(executed.any()):
        return out.to(torch.int32)
    origin = launch_origin(t[:, :, START][executed].numpy())
    for slot in TIME_SLOTS:
        raw = t[:, :, slot]
        ticks = ((raw & 0xFFFFFFFF) - origin) % (1 << 32)
        out[:, :, slot] = torch.where(executed & (raw != 0), ticks, torch.zeros_like(ticks))
    for slot in REFERENCE_ONLY_STAGES:
        out[:, :, slot] = out[:, :, START]
    out[:, :, OPCODE] = torch.where(executed, t[:, :, OPCODE], torch.zeros_like(t[:, :, OPCODE]))
    return out.to(torch.int32)


def microseconds(timings: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """``(t, stamped)``: the records as microseconds since the launch's first instruction started, and
    which slots were stamped at all."""
    raw = timings.astype(np.int64)
    executed = raw[:, :, OPCODE] != 0
    origin = np.int64(launch_origin(raw[:, :, START][executed]))
    t = ((raw & 0xFFFFFFFF) - origin) % (1 << 32) / 100.0
    return t, raw != 0


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

    raw = globs.timings.cpu().numpy()
    ins = globs.instructions.cpu().numpy()
    t, stamped = microseconds(raw)
    op_of = raw[:, :, OPCODE]
    if opts["out"]:
        np.savez_compressed(opts["out"], timings=raw, instructions=ins,
                            reference_layout=reference_event_layout(globs.timings, globs.instructions).numpy(),
                            ticks_per_microsecond=np.array(100))
    print(f"{opts['model']}, {opts['layers']} layers, position {pos}, {partitions} attention partitions, {workers} workers, "
          f"assignment {opts['sched']}: kernel {start.elapsed_time(end) * 1e3:.1f} us with timing records on, "
          f"last instruction ends at {t[:, :, END][op_of != 0].max():.1f} us")
    print("\nper instruction kind, mean / max over all instructions (us); the write back is split into: epilogue "
          "computed and stores issued | stores acknowledged | signalled | workgroup moves on:")
    print(f"{'kind':10s} {'count':>6s} {'wait for dependency':>20s} {'activation':>14s} {'rows':>14s} {'write back':>14s}"
          f" {'issue':>13s} {'ack':>13s} {'signal':>13s} {'leave':>13s}")
    cell = lambda a: f"{a.mean():6.2f} /{a.max():6.2f}" if a.size else "      -"
    for op, name in NAMES.items():
        sel = op_of == op
        if not sel.any():
            continue
        st, dep, inp, rows, done = (t[:, :, i][sel] for i in (START, DEP_READY, INPUT_READY, COMPUTE_DONE, END))
        if op in (2, 3):
            inp = dep  # these record no separate activation event
        line = (f"{name:10s} {int(sel.sum()):6d} {cell(dep - st):>20s} {cell(inp - dep):>14s} {cell(rows - inp):>14s} "
                f"{cell(done - rows):>14s}")
        full = sel & stamped[:, :, AT_GMEM_STORE] & stamped[:, :, DONE_GMEM_STORE] & stamped[:, :, OUTPUT_READY]
        if full.any() and op not in (2, 3):
            issue, ack, sig = (t[:, :, i][full] for i in (AT_GMEM_STORE, DONE_GMEM_STORE, OUTPUT_READY))
            line += (f" {cell(issue - t[:, :, COMPUTE_DONE][full]):>13s} {cell(ack - issue):>13s} {cell(sig - ack):>13s} "
                     f"{cell(t[:, :, END][full] - sig):>13s}")
        print(line)
    layer = min(opts["layer"], opts["layers"] - 1)
    q = lambda a, ps: " ".join(f"{np.percentile(a, p):7.2f}" for p in ps)
    print(f"\nlayer {layer}, over the workers that run the kind (us): first start | dependency seen p10 p50 max | "
          f"last row done (slowest wave) p50 max | signalled p50 max | end p50 max")
    for op in range(1, 7):
        sel = (ins[:, :, 0] == op) & (ins[:, :, 1] == layer)
        if not sel.any():
            continue
        st, dep, done = t[:, :, START][sel], t[:, :, DEP_READY][sel], t[:, :, END][sel]
        waves = np.stack([np.where(stamped[:, :, CONSUMER_START + 2 * w + 1], t[:, :, CONSUMER_START + 2 * w + 1], 0.0)[sel]
                          for w in range(CONSUMER_WAVES)]).max(axis=0)
        sig = np.where(stamped[:, :, OUTPUT_READY], t[:, :, OUTPUT_READY], t[:, :, END])[sel]
        waves = np.where(waves > 0, waves, t[:, :, COMPUTE_DONE][sel])
        print(f"  {NAMES[op]:10s} {st.min():7.2f} | {q(dep, (10, 50, 100))} | {q(waves, (50, 100))} | {q(sig, (50, 100))} | "
              f"{q(done, (50, 100))}")
    sel = ins[:, :, 0] == 7
    if sel.any():
        print(f"  {'lm-head':10s} {t[:, :, START][sel].min():7.2f} | {np.percentile(t[:, :, DEP_READY][sel], 50):7.2f} (p50) | "
              f"{t[:, :, END][sel].max():7.2f} (max)")
    # per layer period: from one layer's QKV dependency (median worker) to the next one's
    deps = [np.percentile(t[:, :, DEP_READY][(ins[:, :, 0] == 1) & (ins[:, :, 1] == l)], 50) for l in range(opts["layers"])]
    if len(deps) > 2:
        print(f"\nlayer period (QKV dependency seen, median worker, layer to layer): mean {np.mean(np.diff(deps[1:])):.2f} us")


if __name__ == "__main__":
    main(sys.argv[1:])

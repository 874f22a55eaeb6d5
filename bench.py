"""Headline benchmark: batch-1 greedy decode through the HIP megakernel.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1..c5] [--extras all|none]

One "step" is one decode step (one token): embedding row -> hidden state,
barrier reset, the instruction stream, argmax over the logits, token write -
the per-token loop of the reference's mk generator
(megakernels/generators.py:121-163).  By default all of it happens inside the
megakernel, and one launch covers --launch-steps consecutive steps (--loop
fused); --launch-steps 1 is one launch per token, and --loop reference runs the
reference's sequence of small kernels around a launch per token instead.
Weights, KV cache and instruction tensor are resident in HBM before the timed
region starts.

Workloads (random bf16 weights N(0, 0.02) from seed 0, RMSNorm weights 1):
  c1  Llama-3.2-1B architecture, 32-token prompt prefilled by the plain PyTorch forward, decode from position 32
  c2  1B, KV cache pre-filled to 4096 positions with seeded N(0,1), decode from position 4096  (default)
  c3  1B, KV cache pre-filled to 16384 positions
  c4  Llama-3.1-8B architecture (untied LM head), 32-token prompt, decode from position 32
  c5  8B, KV cache pre-filled to 32768 positions
The 1B weights come from the CPU generator; the 8B weights (7.5 G parameters) and the long KV
pre-fills are drawn by the GPU's generator, which takes seconds instead of minutes.  The prompt
prefill runs on the GPU, outside the timed region, and its cache is what the CPU checker starts from.

Without --workload the headline line is c2 (the configuration the metric is quoted on) and the other
four workloads are measured in the same process, briefly (--extra-steps timed steps, --extra-cpu-steps
steps checked on the CPU), into the `workloads` object of the line: tokens/s, step time, roofline
fraction and token parity of each; an extra that fails leaves its error string there and the headline
line is printed all the same.  --workload X measures X alone, in full.

Prints one JSON line.  `roofline` prices the megakernel alone: algorithmic
bytes per launch (weights + norm weights + K/V read, summed over the steps of
the launch) divided by the mean launch duration measured with events on the
launch stream.  `cpu_baseline` is the
C restatement of the reference's Python VM (the parity checker) timed on this
host's cores over a bounded number of the same decode steps; its tokens are
also compared with the GPU's.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0

# prefill: cached positions when decoding starts; kv: where they come from
WORKLOADS = {
    "c1": {"arch": "1b", "prefill": 32, "kv": "prompt"},
    "c2": {"arch": "1b", "prefill": 4096, "kv": "random"},
    "c3": {"arch": "1b", "prefill": 16384, "kv": "random"},
    "c4": {"arch": "8b", "prefill": 32, "kv": "prompt"},
    "c5": {"arch": "8b", "prefill": 32768, "kv": "random"},
}


def algorithmic_bytes(cfg, pos: int) -> int:
    """Bytes one decode step must read at least: bf16 matrices (tied embedding
    counted once as the LM head), norm weights, and K/V of positions 0..pos.
    Left out: embedding row, KV append, logits write, rope row, activations,
    instructions, barriers."""
    L, hid, inter = cfg.num_hidden_layers, cfg.hidden_size, cfg.intermediate_size
    H, KVH, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    matrices = L * ((H + 2 * KVH) * D * hid + hid * hid + 3 * inter * hid) + cfg.vocab_size * hid
    norms = (2 * L + 1) * hid
    kv = L * 2 * KVH * D * (pos + 1)
    return 2 * (matrices + norms + kv)


def run_workload(name: str, args, steps: int, warmup: int, cpu_steps: int, torch_steps: int) -> dict:
    """One workload: build the model, schedule and generator, time `steps` decode steps after `warmup`,
    check the first tokens against the CPU checker.  Returns the JSON object of the workload."""
    import torch

    from megakernels_amd.demos.latency.scheduler import LatencyScheduleBuilder, pick_num_attention_partitions
    from megakernels_amd.dispatch import make_mk_interpreter
    from megakernels_amd.generators import MK_Generator
    from megakernels_amd.llama import LlamaConfig, LlamaForCausalLM
    from megakernels_amd.model_types import BatchState, ExtraModelConfig
    from megakernels_amd.scheduler import assign_to_sms, tensorize_instructions
    from megakernels_amd.utils import get_sm_count, set_sm_count_override

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    work = WORKLOADS[name]
    big = work["arch"] == "8b"
    cfg = LlamaConfig.llama_8b() if big else LlamaConfig.llama_1b()
    total_steps = warmup + steps
    prefill = work["prefill"]
    max_len = prefill + total_steps + 16
    if cpu_steps < 0:
        cpu_steps = 4 if big else 32
    if torch_steps < 0:
        torch_steps = 1 if big else 3
    need_cpu_twin = cpu_steps > 0 or torch_steps > 0
    t_setup = time.time()
    extra = ExtraModelConfig(interleave_rope=True, max_len_override=max_len)
    if big:
        model = LlamaForCausalLM.from_random(cfg, extra, seed=0, device=device, draw_device=device)
        model_cpu = model.to("cpu") if need_cpu_twin else None
    else:
        model_cpu = LlamaForCausalLM.from_random(cfg, extra, seed=0)
        model = model_cpu.to(device)

    prompt_gen = torch.Generator().manual_seed(1)
    prompt = torch.randint(0, cfg.vocab_size, (1, 32), generator=prompt_gen)
    if work["kv"] == "prompt":
        # prefill once with the plain forward on the GPU (reference scripts/generate.py:125-137); the
        # megakernel and the checker both start from its cache
        out = model(BatchState(input_ids=prompt.to(device), position_ids=torch.arange(32, device=device)))
        first_token = int(out.output_ids[0, -1])
    else:
        kv_gen = torch.Generator(device=device).manual_seed(2)
        for cache in model.stacked_kv_cache:
            for layer in range(cache.shape[0]):
                rows = torch.randn((cache.shape[1], prefill) + tuple(cache.shape[3:]), generator=kv_gen, device=device)
                cache[layer, :, :prefill] = rows.to(cache.dtype)
        first_token = int(prompt[0, 0])
    if model_cpu is not None:
        for dst, src in zip(model_cpu.stacked_kv_cache, model.stacked_kv_cache):
            dst.copy_(src)

    workers = args.workers or get_sm_count(device)
    set_sm_count_override(workers)
    partitions = args.partitions or pick_num_attention_partitions(prefill, total_steps, device, cfg.num_key_value_heads, cfg.head_dim)

    schedule = LatencyScheduleBuilder.build(model, num_attention_partitions=partitions)
    tensorize_instructions(schedule.globs, assign_to_sms(args.sched, schedule=schedule))
    interpreter = make_mk_interpreter("latency")
    gen = MK_Generator(model, interpreter, schedule, fused_step=args.loop == "fused",
                       steps_per_launch=args.launch_steps if args.loop == "fused" else 1)
    mk_mod = sys.modules["mk_llama"]

    ntok = total_steps + 1
    output_tokens = torch.zeros(1, ntok, device=device, dtype=torch.long)
    output_tokens[0, 0] = first_token
    torch.cuda.synchronize()
    setup_s = time.time() - t_setup

    # ---- warmup -------------------------------------------------------------
    if warmup:
        gen.generate(output_tokens, prompt_len=prefill, ntok=warmup, ntok_already_generated=1)
    torch.cuda.synchronize()
    mk_mod.check_status(device)

    # ---- timed region: exactly K steps --------------------------------------
    # kernel-only events: wrap the interpreter so each launch is bracketed on the launch stream
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    steps_of_launch = []
    plain = {n: getattr(interpreter, n) for n in ("interpret", "interpret_step", "interpret_steps")}

    def timed(launch, count):
        def wrapper(*a, **kw):
            i = len(steps_of_launch)
            starts[i].record()
            launch(*a, **kw)
            ends[i].record()
            steps_of_launch.append(count(*a, **kw))
        return wrapper

    interpreter.interpret = timed(plain["interpret"], lambda *a, **kw: 1)
    interpreter.interpret_step = timed(plain["interpret_step"], lambda *a, **kw: 1)
    interpreter.interpret_steps = timed(plain["interpret_steps"], lambda globs, embed, token_in, tokens_out: tokens_out.numel())
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    gen.generate(output_tokens, prompt_len=prefill, ntok=steps, ntok_already_generated=1 + warmup)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    for n, fn in plain.items():
        setattr(interpreter, n, fn)
    mk_mod.check_status(device)
    assert sum(steps_of_launch) == steps

    launch_ms = [s.elapsed_time(e) for s, e, _ in zip(starts, ends, steps_of_launch)]
    first_pos = prefill + warmup
    step_bytes = [algorithmic_bytes(cfg, first_pos + i) for i in range(steps)]
    bytes_per_step = sum(step_bytes) / steps
    # the roofline is quoted on the launches of the usual size (a shorter last launch, when the
    # step count does not divide, is left out of the mean)
    usual = max(steps_of_launch)
    usual_ms, usual_bytes, at = [], [], 0
    for ms, n in zip(launch_ms, steps_of_launch):
        if n == usual:
            usual_ms.append(ms)
            usual_bytes.append(sum(step_bytes[at : at + n]))
        at += n
    kernel_ms_mean = sum(usual_ms) / len(usual_ms)
    bytes_per_launch = sum(usual_bytes) / len(usual_bytes)
    achieved_gbps = bytes_per_launch / (kernel_ms_mean * 1e-3) / 1e9

    tokens_gpu = output_tokens[0].cpu().tolist()

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)   # elementwise copy kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    # ---- CPU baseline: the checker on the same decode steps (bounded sample) --
    cpu_baseline = None
    parity = None
    if cpu_steps > 0:
        from oracle import pyvm

        n_cpu = min(cpu_steps, total_steps)
        set_sm_count_override(workers)
        schedule_cpu = LatencyScheduleBuilder.build(model_cpu, num_attention_partitions=partitions)
        oracle_gen = pyvm.OracleGenerator(model_cpu, schedule_cpu)
        tokens_cpu = torch.zeros(1, n_cpu + 1, dtype=torch.long)
        tokens_cpu[0, 0] = first_token
        tc0 = time.perf_counter()
        oracle_gen.generate(tokens_cpu, prompt_len=prefill, ntok=n_cpu, ntok_already_generated=1)
        cpu_elapsed = time.perf_counter() - tc0
        cpu_baseline = {
            "value": round(n_cpu / cpu_elapsed, 3),
            "unit": "tokens/s",
            "cores": pyvm.threads(),
            "kind": "port",
            "sample": f"first {n_cpu} decode steps of the same workload on the C restatement of the Python VM "
                      f"(OpenMP, {pyvm.threads()} threads), {cpu_elapsed:.1f} s",
            "us_per_step": round(cpu_elapsed / n_cpu * 1e6, 1),
        }
        expect = tokens_cpu[0].tolist()
        got = tokens_gpu[: n_cpu + 1]
        agree = sum(int(a == b) for a, b in zip(expect, got))
        parity = {"tokens_compared": n_cpu + 1, "tokens_equal": agree, "bit_exact": agree == n_cpu + 1}
        if torch_steps > 0:
            # the same steps once more on the restatement written with the reference's own torch calls
            # (one small bf16 matvec per 16-row block, as megakernels/demos/latency/python_vm.py does):
            # what the reference's Python VM costs on these cores
            from oracle import pyvm_torch

            n_torch = min(torch_steps, n_cpu)
            globs = schedule_cpu.globs
            instructions = schedule_cpu.get_linear_instructions()
            embed = model_cpu.model.embed_tokens.weight
            for dst, src in zip(model_cpu.stacked_kv_cache, model.stacked_kv_cache):
                dst.copy_(src)   # the checker appended rows; start from the same cache again
            tt0 = time.perf_counter()
            for i in range(n_torch):
                globs.hidden_states[:] = embed[int(tokens_cpu[0, i])]
                globs.barriers.zero_()
                globs.pos_id = prefill + i
                pyvm_torch.interpret(globs, instructions)
            torch_elapsed = time.perf_counter() - tt0
            cpu_baseline["torch_restatement"] = {
                "value": round(n_torch / torch_elapsed, 4),
                "unit": "tokens/s",
                "cores": torch.get_num_threads(),
                "kind": "torch-restatement",
                "sample": f"first {n_torch} decode step(s), torch.set_num_threads default ({torch.get_num_threads()}), "
                          f"{torch_elapsed:.1f} s",
                "us_per_step": round(torch_elapsed / n_torch * 1e6, 1),
            }

    # HBM bytes per launch measured with rocprofv3 --pmc for this workload (committed summary)
    traffic = None
    traffic_source = None
    traffic_file = ROOT / "profiles" / f"mk_llama_kernel_{name}_traffic.json"
    if traffic_file.exists():
        traffic_source = f"committed rocprofv3 --pmc summary profiles/{traffic_file.name} (not measured in this run)"
        measured = json.loads(traffic_file.read_text())
        # the counters were taken per launch of `steps_per_launch` steps
        per_step = (measured["fetch_bytes_per_launch"] + measured["write_bytes_per_launch"]) / measured.get("steps_per_launch", 1)
        traffic = int(per_step * usual)

    return {
        "metric": f"batch-1 decode tokens/s ({'Llama-3.1-8B' if big else 'Llama-3.2-1B'} arch)",
        "value": round(steps / elapsed, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(elapsed / steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{name}: {'Llama-3.1-8B' if big else 'Llama-3.2-1B'} architecture, random-init bf16 "
                        f"weights (seed 0, {'GPU' if big else 'CPU'} generator), batch 1, "
                        + (f"32-token prompt prefilled on the GPU, " if work["kv"] == "prompt" else
                           f"KV pre-filled to {prefill} positions with seeded N(0,1), ")
                        + f"greedy decode of {steps} timed tokens from position {first_pos}",
            "workers": workers,
            "attention_partitions": partitions,
            "assignment": args.sched,
            "loop": args.loop,
            "steps_per_launch": usual,
            "instructions_per_step": len(schedule.dag_nodes),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved_gbps / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel": "mk_llama_kernel<8,4,128,false>" if big else "mk_llama_kernel<4,4,64,false>",
            "kernel_us": round(kernel_ms_mean * 1e3, 2),
            "kernel_us_per_step": round(kernel_ms_mean * 1e3 / usual, 2),
            "launches_timed": len(usual_ms),
            "algorithmic_bytes_per_launch": int(bytes_per_launch),
        },
        "cpu_baseline": cpu_baseline,
        "parity": parity,
        "whole_step_roofline_frac": round(bytes_per_step / (elapsed / steps) / 1e9 / HBM_PEAK_GBPS, 4),
        "setup_s": round(setup_s, 1),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help="the workload of the headline line (default c2, the one the metric is quoted on); given "
                         "explicitly, only that workload runs")
    ap.add_argument("--extras", default=None, choices=["all", "none"],
                    help="also measure the other four workloads of the baseline, briefly, into the `workloads` object "
                         "of the same JSON line (default: all when --workload is not given)")
    ap.add_argument("--extra-steps", type=int, default=16, help="timed decode steps of each extra workload")
    ap.add_argument("--extra-cpu-steps", type=int, default=2, help="decode steps of each extra workload checked on the CPU")
    ap.add_argument("--cpu-steps", type=int, default=-1,
                    help="decode steps timed on the CPU checker (0 = skip; default 32 for the 1B workloads, 4 for 8B)")
    ap.add_argument("--torch-steps", type=int, default=-1,
                    help="decode steps also timed on the torch restatement of the Python VM, the closer stand-in for "
                         "the reference's python_vm.py (0 = skip; default 3 for 1B, 1 for 8B)")
    ap.add_argument("--sched", default="rr")
    ap.add_argument("--workers", type=int, default=0, help="instruction queues (0 = one per compute unit)")
    ap.add_argument("--partitions", type=int, default=0, help="attention partitions (0 = one per 256 positions, at most 24, or one per worker and KV head when the jobs are long)")
    ap.add_argument("--loop", default="fused", choices=["fused", "reference"],
                    help="fused: one launch per token (embedding row, barrier reset and argmax inside the "
                         "megakernel); reference: the reference generator's sequence of small kernels around "
                         "the launch")
    ap.add_argument("--launch-steps", type=int, default=8,
                    help="--loop fused: decode steps per megakernel launch (the token of one step starts the "
                         "next inside the kernel); 1 = one launch per token, 0 = all steps of a phase in one launch")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="after the timed region also run a plain 1 GiB device copy three times, so that a "
                         "rocprofv3 --pmc run of this command holds a kernel of known traffic to scale "
                         "FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the decode path on ONE GPU; --gpus N with N > 1 is not supported "
              "(batch-1 decode does not shard into independent units)", file=sys.stderr)
        sys.exit(2)

    import gc

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    headline = args.workload or "c2"
    extras = args.extras or ("all" if args.workload is None else "none")
    result = run_workload(headline, args, args.steps, args.warmup, args.cpu_steps, args.torch_steps)
    if extras == "all":
        # the other workloads of the baseline in the same process, briefly: the figures a reader needs
        # to place them (throughput, step time, roofline fraction, token parity), not the full record
        result["workloads"] = {}
        for name in sorted(WORKLOADS):
            if name == headline:
                continue
            gc.collect()
            torch.cuda.empty_cache()
            try:
                extra_steps = max(args.launch_steps, args.extra_steps)
                r = run_workload(name, args, extra_steps, max(args.launch_steps, 8), args.extra_cpu_steps, 0)
                result["workloads"][name] = {
                    "workload": r["config"]["workload"],
                    "value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"],
                    "steps": r["steps"], "attention_partitions": r["config"]["attention_partitions"],
                    "roofline": {"frac": r["roofline"]["frac"], "achieved": r["roofline"]["achieved"], "unit": "GB/s",
                                 "kernel": r["roofline"]["kernel"], "kernel_us_per_step": r["roofline"]["kernel_us_per_step"],
                                 "launches_timed": r["roofline"]["launches_timed"]},
                    "cpu_baseline": {k: r["cpu_baseline"][k] for k in ("value", "unit", "cores", "kind", "sample")} if r["cpu_baseline"] else None,
                    "parity": r["parity"],
                    "setup_s": r["setup_s"],
                }
            except Exception as e:  # the headline line is printed whatever happens to an extra
                result["workloads"][name] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()

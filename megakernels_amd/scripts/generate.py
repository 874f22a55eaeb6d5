"""Decode benchmark / demo entry point with the argument surface of the reference's
``megakernels/scripts/generate.py`` (``key=value`` pairs, presets written ``.name``):

    python -m megakernels_amd.scripts.generate mode=mk ntok=100
    python -m megakernels_amd.scripts.generate .l8 mode=mk prompt_len=32 ntok=64 num_attention_partitions=4

Differences forced by the environment: nothing is downloaded, so ``model`` is ``1b`` / ``8b``
(random-initialised architecture; the prompt is ``prompt_len`` seeded random token ids) or a local checkpoint
directory; when that directory holds a tokenizer, ``prompt=...`` (``chat=true`` for the chat template) is
tokenised and the output is printed as text too, as the reference does (``generate.py:98-112,186-202``).  Modes: ``mk`` (HIP megakernel) and ``torch`` (plain PyTorch forward).
As in the reference (``generate.py:125-137``) the prompt is prefilled by the PyTorch model and the timed
region is ``ntok - 1`` decode steps, repeated ``num_warmup + num_iters`` times.
"""

from __future__ import annotations

import sys
import time
from dataclasses import dataclass, fields
from pathlib import Path

import torch

from megakernels_amd.dispatch import make_mk_interpreter, make_schedule_builder
from megakernels_amd.generators import MK_Generator, PyTorchGenerator
from megakernels_amd.llama import LlamaConfig, LlamaForCausalLM
from megakernels_amd.mk import DEFAULT_MK_DIR
from megakernels_amd.model_types import BatchState, ExtraModelConfig
from megakernels_amd.scheduler import assign_to_sms, tensorize_instructions
from megakernels_amd.scripts.text import encode_prompt, load_tokenizer


@dataclass
class ScriptConfig:
    model: str = "1b"
    device: str = "cuda:0"
    prompt: str = "tell me a funny joke about cookies"
    chat: bool = False
    token_details: bool = False
    prompt_len: int = 32
    ntok: int = 100
    mode: str = "mk"
    interleave_rope: bool = True
    mk_dir: Path = DEFAULT_MK_DIR
    tokens: bool = True
    num_warmup: int = 5
    num_iters: int = 10
    barrier_fill_val: int = 0
    max_len_override: int | None = 16384
    noops: bool = False
    skip_mk: bool = False
    skip_rest: bool = False
    sched: str = "rr"
    setting: str = "latency"
    memory_fraction: float | None = None
    num_attention_partitions: int = 1
    seed: int = 0

    # presets, selected on the command line as `.name`
    def once(self):
        self.num_warmup, self.num_iters = 0, 1

    def l1(self):
        self.model = "1b"

    def l8(self):
        self.model = "8b"

    def finalize(self):
        if self.mode == "mk":
            assert self.interleave_rope, "interleave_rope must be True for mk mode"
        if self.mode == "pyvm":
            raise SystemExit("mode=pyvm: the Python VM is a test-only checker in this build (see oracle/)")


def parse_args(argv: list[str]) -> ScriptConfig:
    cfg = ScriptConfig()
    types = {f.name: f.type for f in fields(cfg)}
    for arg in argv:
        if arg.startswith("."):
            getattr(cfg, arg[1:])()
            continue
        key, _, value = arg.partition("=")
        if key not in types:
            raise SystemExit(f"unknown argument {key!r}")
        current = getattr(cfg, key)
        if value in ("None", "none"):
            parsed = None
        elif isinstance(current, bool):
            parsed = value.lower() in ("1", "true", "t", "yes")
        elif isinstance(current, int) or "int" in str(types[key]):
            parsed = int(value)
        elif isinstance(current, float) or "float" in str(types[key]):
            parsed = float(value)
        elif isinstance(current, Path):
            parsed = Path(value)
        else:
            parsed = value
        setattr(cfg, key, parsed)
    cfg.finalize()
    return cfg


def load_model(config: ScriptConfig) -> LlamaForCausalLM:
    extra = ExtraModelConfig(interleave_rope=config.interleave_rope, max_len_override=config.max_len_override)
    if config.model in ("1b", "8b"):
        arch = LlamaConfig.llama_1b() if config.model == "1b" else LlamaConfig.llama_8b()
        return LlamaForCausalLM.from_random(arch, extra, seed=config.seed, device=config.device)
    return LlamaForCausalLM.from_pretrained(config.model, extra, device=config.device)


@torch.inference_mode()
def main(config: ScriptConfig):
    torch.cuda.set_device(config.device)
    model = load_model(config)
    tokenizer = None if config.model in ("1b", "8b") else load_tokenizer(config.model)
    if tokenizer is not None:
        input_ids = encode_prompt(tokenizer, config.prompt, config.chat).to(model.device)
    else:
        gen_ids = torch.Generator().manual_seed(config.seed + 1)
        input_ids = torch.randint(0, model.config.vocab_size, (1, config.prompt_len), generator=gen_ids).to(model.device)
    prompt_len = input_ids.shape[-1]
    print(f"Input ids shape: {tuple(input_ids.shape)}")

    prefill = model(BatchState(input_ids=input_ids, position_ids=torch.arange(prompt_len, device=model.device)))
    output_tokens = torch.zeros(1, config.ntok, device=model.device, dtype=torch.long)
    output_tokens[:, 0] = prefill.output_ids[:, -1]

    builder = make_schedule_builder(config.setting)
    schedule = builder.build(model, num_attention_partitions=config.num_attention_partitions)
    queues = assign_to_sms(config.sched, schedule=schedule, memory_fraction=config.memory_fraction)
    tensorize_instructions(schedule.globs, queues)

    if config.mode == "torch":
        gen = PyTorchGenerator(model)
    elif config.mode == "mk":
        interpreter = make_mk_interpreter(config.setting, config.mk_dir)
        gen = MK_Generator(model, interpreter, schedule, barrier_fill_val=config.barrier_fill_val,
                           skip_mk=config.skip_mk, skip_rest=config.skip_rest)
        if config.noops:
            gen.replace_with_noops()
    else:
        raise ValueError(f"Invalid mode: {config.mode}")

    times, cpu_times = [], []
    for _ in range(config.num_warmup + config.num_iters):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        t0 = time.time()
        gen.generate(output_tokens, prompt_len, config.ntok - 1)
        t1 = time.time()
        end.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(end) / 1000)
        cpu_times.append(t1 - t0)
    if config.mode == "mk":
        sys.modules["mk_llama"].check_status(config.device)

    elapsed = sum(times[config.num_warmup:]) / config.num_iters
    elapsed_cpu = sum(cpu_times[config.num_warmup:]) / config.num_iters
    print(f"Average time: {elapsed * 1000:.2f}ms (CPU: {elapsed_cpu * 1000:.2f}ms)")
    if config.tokens:
        print("Output ids: ", output_tokens.cpu())
        if tokenizer is not None:
            print("Output text: ", tokenizer.batch_decode(output_tokens.cpu()))
    if config.token_details and tokenizer is not None:
        print("More detailed output (output id, position id, token):")
        for i, token in enumerate(tokenizer.convert_ids_to_tokens(output_tokens[0].cpu().tolist())):
            print(f"  {i:5d} {i + prompt_len:6d}  {token}")
    fwd_per_second = (config.ntok - 1) / elapsed
    print(f"Fwd per second: {fwd_per_second:.2f}")
    print(f"Tokens per second: {fwd_per_second:.2f}")
    return output_tokens


if __name__ == "__main__":
    main(parse_args(sys.argv[1:]))

"""Chat with a local Llama checkpoint through the megakernel (reference ``scripts/llama_repl.py``).

    python -m megakernels_amd.scripts.llama_repl model=/path/to/Llama-3.2-1B-Instruct [mode=mk|torch]
        [max_tokens_per_turn=1024] [sched=rr] [num_attention_partitions=1] [print_prompt_len=true]

Every turn renders the whole conversation through the tokenizer's chat template, prefills it with the
plain PyTorch forward, then decodes greedily until an end-of-sequence id (looked for on the host every 16
tokens, which is also how many decode steps go into one launch) or ``max_tokens_per_turn``.  The directory
must hold ``config.json``, ``*.safetensors`` and the tokenizer; nothing is downloaded.
"""

from __future__ import annotations

import sys
import time
from dataclasses import dataclass, fields
from pathlib import Path

import torch

from megakernels_amd.dispatch import make_mk_interpreter, make_schedule_builder
from megakernels_amd.generators import Generator, MK_Generator, PyTorchGenerator
from megakernels_amd.llama import LlamaForCausalLM
from megakernels_amd.mk import DEFAULT_MK_DIR
from megakernels_amd.model_types import BatchState, ExtraModelConfig
from megakernels_amd.scheduler import assign_to_sms, tensorize_instructions
from megakernels_amd.scripts.text import encode_messages, eos_token_ids, load_tokenizer

EOS_CHECK_INTERVAL = 16


@dataclass
class ScriptConfig:
    model: str = ""
    device: str = "cuda:0"
    max_tokens_per_turn: int = 1024
    mk_dir: Path = DEFAULT_MK_DIR
    mode: str = "mk"
    sched: str = "rr"
    setting: str = "latency"
    memory_fraction: float | None = None
    num_attention_partitions: int = 1
    print_prompt_len: bool = False


def parse_args(argv: list[str]) -> ScriptConfig:
    cfg = ScriptConfig()
    known = {f.name: f.type for f in fields(cfg)}
    for arg in argv:
        key, _, value = arg.partition("=")
        if key not in known:
            raise SystemExit(f"unknown argument {key!r}; known: {', '.join(known)}")
        current = getattr(cfg, key)
        if isinstance(current, bool):
            setattr(cfg, key, value.lower() in ("1", "true", "t", "yes"))
        elif isinstance(current, int):
            setattr(cfg, key, int(value))
        elif isinstance(current, Path):
            setattr(cfg, key, Path(value))
        elif key == "memory_fraction":
            setattr(cfg, key, None if value in ("None", "none") else float(value))
        else:
            setattr(cfg, key, value)
    if not cfg.model:
        raise SystemExit("model=<local checkpoint directory> is required (nothing is downloaded)")
    return cfg


class Conversation:
    """The state of one chat: model, generator, token buffer, messages so far."""

    def __init__(self, model: LlamaForCausalLM, gen: Generator, tokenizer, eos_ids: list[int],
                 max_tokens_per_turn: int, print_prompt_len: bool = False):
        self.model, self.gen, self.tokenizer, self.eos_ids = model, gen, tokenizer, eos_ids
        self.max_tokens_per_turn = max_tokens_per_turn
        self.print_prompt_len = print_prompt_len
        self.output_tokens = torch.zeros(1, max_tokens_per_turn, device=model.device, dtype=torch.long)
        self.messages: list[dict] = []

    @torch.inference_mode()
    def respond(self, messages: list[dict]) -> tuple[str, int, float]:
        """Answer to ``messages``: ``(text, decode steps run, seconds spent decoding)``."""
        input_ids = encode_messages(self.tokenizer, messages).to(self.model.device)
        prompt_len = input_ids.shape[-1]
        if self.print_prompt_len:
            print(f"Prompt length: {prompt_len}")
        if prompt_len + self.max_tokens_per_turn > self.model.stacked_kv_cache[0].shape[2]:
            raise RuntimeError(f"a prompt of {prompt_len} tokens plus {self.max_tokens_per_turn} new ones does not "
                               "fit the KV cache")
        prefill = self.model(BatchState(input_ids=input_ids, position_ids=torch.arange(prompt_len, device=self.model.device)))
        self.output_tokens[:, 0] = prefill.output_ids[:, -1]
        if self.model.device.type == "cuda":
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        # looks at the tokens on the host after every chunk, so the clock can stop right after it
        until_eos, generated = self.gen.generate_with_eos(
            output_tokens=self.output_tokens, prompt_len=prompt_len, ntok=self.max_tokens_per_turn,
            eos_token_ids=self.eos_ids, eos_token_check_interval=EOS_CHECK_INTERVAL)
        seconds = time.perf_counter() - t0
        text = self.tokenizer.decode(self.output_tokens[0, :until_eos].cpu(), skip_special_tokens=True)
        return text, generated, seconds

    def say(self, user_input: str) -> tuple[str, int, float]:
        self.messages.append({"role": "user", "content": user_input})
        text, generated, seconds = self.respond(self.messages)
        self.messages.append({"role": "assistant", "content": text})
        return text, generated, seconds


def build_conversation(config: ScriptConfig) -> Conversation:
    tokenizer = load_tokenizer(config.model)
    if tokenizer is None:
        raise SystemExit(f"no tokenizer under {config.model}")
    model = LlamaForCausalLM.from_pretrained(config.model, ExtraModelConfig(interleave_rope=True, max_batch_size=1),
                                             device=config.device)
    if config.mode == "torch":
        gen: Generator = PyTorchGenerator(model)
    elif config.mode == "mk":
        schedule = make_schedule_builder(config.setting).build(model, num_attention_partitions=config.num_attention_partitions)
        tensorize_instructions(schedule.globs, assign_to_sms(config.sched, schedule=schedule, memory_fraction=config.memory_fraction))
        gen = MK_Generator(model, make_mk_interpreter(config.setting, config.mk_dir), schedule)
    else:
        raise SystemExit(f"invalid mode {config.mode!r}: mk or torch")
    return Conversation(model, gen, tokenizer, eos_token_ids(config.model, tokenizer), config.max_tokens_per_turn,
                        config.print_prompt_len)


def main(config: ScriptConfig):
    if config.device.startswith("cuda"):
        torch.cuda.set_device(config.device)
    chat = build_conversation(config)
    chat.respond([{"role": "user", "content": "hi"}])  # warm-up
    print("the megakernel is listening (ctrl-d to leave)")
    while True:
        try:
            user_input = input(">>> ")
        except EOFError:
            print()
            return
        text, generated, seconds = chat.say(user_input)
        print("Response: ", text)
        print(f"Speed: {generated / seconds:.2f} tokens/s")


if __name__ == "__main__":
    main(parse_args(sys.argv[1:]))

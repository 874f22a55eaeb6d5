"""Text in and out for the scripts: tokenizer of a local checkpoint directory, prompt encoding with
or without the chat template, end-of-sequence ids (what the reference's scripts do inline with
``transformers``: ``scripts/generate.py:86,98-112``, ``scripts/llama_repl.py:36-41,85-92``).

Nothing is downloaded: the tokenizer must sit next to the weights.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch


def load_tokenizer(model_dir: str | Path):
    """The tokenizer stored in ``model_dir``, or None when the directory holds none."""
    path = Path(model_dir)
    if not path.is_dir() or not any((path / name).exists() for name in ("tokenizer.json", "tokenizer.model")):
        return None
    from transformers import AutoTokenizer

    return AutoTokenizer.from_pretrained(str(path), local_files_only=True)


def encode_prompt(tokenizer, prompt: str, chat: bool) -> torch.Tensor:
    """``[1, prompt_len]`` token ids: the bare prompt with the tokenizer's special tokens, or one user
    turn rendered through the chat template followed by the generation prompt."""
    return encode_messages(tokenizer, [{"role": "user", "content": prompt}]) if chat else \
        tokenizer(prompt, return_tensors="pt", add_special_tokens=True)["input_ids"]


def encode_messages(tokenizer, messages: list[dict]) -> torch.Tensor:
    text = tokenizer.apply_chat_template(messages, tokenize=False, add_generation_prompt=True)
    return tokenizer(text, return_tensors="pt", add_special_tokens=False)["input_ids"]


def eos_token_ids(model_dir: str | Path, tokenizer=None) -> list[int]:
    """End-of-sequence ids: ``generation_config.json`` first (a number or a list), then ``config.json``,
    then the tokenizer's own."""
    path = Path(model_dir)
    for name in ("generation_config.json", "config.json"):
        file = path / name
        if file.exists():
            ids = json.loads(file.read_text()).get("eos_token_id")
            if isinstance(ids, int):
                return [ids]
            if isinstance(ids, list) and ids:
                return [int(i) for i in ids]
    if tokenizer is not None and tokenizer.eos_token_id is not None:
        return [int(tokenizer.eos_token_id)]
    return []

"""Shared builders for the parity tests: small seeded models, paired CPU / GPU
buffer bundles, KV prefill, and exact tensor comparison."""

from __future__ import annotations

import torch

from megakernels_amd.demos.latency.scheduler import LatencyScheduleBuilder
from megakernels_amd.llama import LlamaConfig, LlamaForCausalLM
from megakernels_amd.model_types import ExtraModelConfig
from megakernels_amd.scheduler import assign_to_sms, tensorize_instructions
from megakernels_amd.utils import set_sm_count_override


def config_tiny(layers=2):
    """512 wide, 8 query / 2 KV heads of 64: the smallest shape the kernel has an instance for."""
    return LlamaConfig(
        hidden_size=512, intermediate_size=1024, num_hidden_layers=layers, num_attention_heads=8,
        num_key_value_heads=2, head_dim=64, vocab_size=1024, max_position_embeddings=1024,
    )


def config_1b_slice(layers=2, vocab=8192):
    """Llama-3.2-1B layer shapes with fewer layers and a small vocabulary."""
    return LlamaConfig(num_hidden_layers=layers, vocab_size=vocab, max_position_embeddings=8192)


def config_8b_slice(layers=1, vocab=4096, inter=6144):
    """Llama-3.1-8B attention shapes (4096 wide, head_dim 128) with a narrower MLP:
    two O-projection column groups, inter / 2048 down-projection groups."""
    cfg = LlamaConfig.llama_8b()
    cfg.num_hidden_layers = layers
    cfg.vocab_size = vocab
    cfg.intermediate_size = inter
    cfg.max_position_embeddings = 8192
    return cfg


def make_model(cfg, max_len=256, seed=0):
    return LlamaForCausalLM.from_random(
        cfg, ExtraModelConfig(interleave_rope=True, max_len_override=max_len), seed=seed
    )


def fill_kv(model, upto: int, seed=2, poison=True):
    """Seeded N(0,1) K/V for positions [0, upto); N(0,100) beyond, as the reference's
    diff_test.py:106-118 does, so that reading past the sequence shows up."""
    gen = torch.Generator().manual_seed(seed)
    for cache in model.stacked_kv_cache:
        shape = list(cache.shape)
        cache.copy_(torch.randn(shape, generator=gen).to(cache.dtype))
        if poison:
            tail = torch.randn(shape, generator=gen) * 100
            cache[:, :, upto:] = tail[:, :, upto:].to(cache.dtype)
        else:
            cache[:, :, upto:] = 0


def make_model_pair(cfg, max_len, seed=0, device="cuda:0"):
    """(CPU model, GPU model) with identical weights drawn by the GPU's generator: the full-size
    architectures take seconds this way and minutes with the CPU generator."""
    model_gpu = LlamaForCausalLM.from_random(
        cfg, ExtraModelConfig(interleave_rope=True, max_len_override=max_len), seed=seed, device=device, draw_device=device
    )
    return model_gpu.to("cpu"), model_gpu


def fill_kv_pair(model_cpu, model_gpu, upto: int, seed=2):
    """fill_kv for a model pair: drawn on the GPU, copied to the CPU twin.  Seeded N(0,1) for
    positions [0, upto), N(0,100) beyond."""
    gen = torch.Generator(device=model_gpu.device).manual_seed(seed)
    for dst, twin in zip(model_gpu.stacked_kv_cache, model_cpu.stacked_kv_cache):
        # layer by layer: the fp32 draw of a whole 32k-position cache is a multiple of the cache itself
        for layer in range(dst.shape[0]):
            rows = torch.randn(dst.shape[1:], generator=gen, device=dst.device)
            rows[:, upto:] *= 100
            dst[layer].copy_(rows)
        twin.copy_(dst)


def build_schedule(model, workers, partitions=1, sched="rr", stop_after_op=None, layer_limit=None):
    set_sm_count_override(workers)
    schedule = LatencyScheduleBuilder.build(
        model, stop_after_op=stop_after_op, layer_limit=layer_limit, num_attention_partitions=partitions
    )
    queues = assign_to_sms(sched, schedule=schedule)
    tensorize_instructions(schedule.globs, queues)
    return schedule


def mirror_to_gpu(model_cpu, schedule_cpu, device="cuda:0", model_gpu=None):
    """GPU twin of a CPU model + schedule: same weights, same KV contents, same
    instruction tensor, fresh activation buffers holding the same values.
    ``model_gpu``: an existing twin of the model (weights and KV already equal)."""
    if model_gpu is None:
        model_gpu = model_cpu.to(device)
        for dst, src in zip(model_gpu.stacked_kv_cache, model_cpu.stacked_kv_cache):
            dst.copy_(src)
    workers = schedule_cpu.globs.instructions.shape[0]
    set_sm_count_override(workers)
    gcpu = schedule_cpu.globs
    from dataclasses import replace

    ggpu = LatencyScheduleBuilder.make_globals(model_gpu, skip_attn_reduction=gcpu.skip_attn_reduction)
    schedule_gpu = replace(schedule_cpu, globs=ggpu)
    ggpu.instructions = gcpu.instructions.to(device)
    ggpu.timings = gcpu.timings.to(device)
    for name in ("hidden_states", "post_ln_rope_q", "attn_out", "attn_lse_intermediates",
                 "attn_out_intermediates", "silu_out", "logits", "barriers"):
        getattr(ggpu, name).copy_(getattr(gcpu, name))
    ggpu.pos_id = gcpu.pos_id
    return model_gpu, schedule_gpu


def bits(t: torch.Tensor) -> torch.Tensor:
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16)
    if t.dtype == torch.float32:
        return t.view(torch.int32)
    return t


def mismatches(g_ref, g_dev, names=None, kv_rows=None):
    """{name: count of differing elements} over the mutable tensors.  NaNs
    compare by bit pattern.  ``kv_rows``: only compare these cache positions."""
    report = {}
    for name in names or g_ref.mutable_tensor_names():
        a, b = getattr(g_ref, name), getattr(g_dev, name)
        if kv_rows is not None and "cache" in name:
            a, b = a[:, :, kv_rows], b[:, :, kv_rows]
        n = int((bits(a) != bits(b)).sum())
        if n:
            report[name] = n
    return report


class _Holder:
    def __init__(self, **kw):
        self.__dict__.update(kw)


def shape_only_model(cfg, max_len=64):
    """A stand-in model that carries the architecture and zero-element tensors:
    enough for the scheduler (pure integer logic), far too little to run."""
    empty = torch.empty(0, dtype=torch.bfloat16)
    params = _Holder(qkv_proj=empty, o_proj=empty, attn_ln_weight=empty, mlp_ln_weight=empty,
                     up_proj=empty, gate_proj=empty, down_proj=empty)
    return _Holder(
        config=cfg, device=torch.device("cpu"), dtype=torch.bfloat16, stacked_params=params,
        lm_head=_Holder(input_norm=_Holder(weight=empty), lm_head=_Holder(weight=empty)),
        stacked_kv_cache=(empty, empty), model=_Holder(rope_cos=empty, rope_sin=empty),
    )

"""GPU parity at the real shapes of the five benchmark configurations: the full Llama-3.2-1B
architecture (16 layers, vocabulary 128256) at short context, at 4096 cached positions with 17
attention partitions and at 16384 with 24; the full Llama-3.1-8B architecture (32 layers, MLP 14336 =
seven down-projection column groups, untied LM head) at short context and at 32768 cached positions.

Each case runs one decode step from a random hidden state and compares every buffer the VM writes,
bit for bit, with the C restatement of the reference's Python VM (python_vm.py:83-393 semantics); the
decode cases then generate a few tokens through the fused loop and compare token ids and the KV rows
written.  Weights are drawn on the GPU (seconds instead of minutes) and copied to the checker."""

import sys

import pytest
import torch

from helpers import build_schedule, fill_kv_pair, make_model_pair, mirror_to_gpu, mismatches

pytestmark = pytest.mark.gpu


def _interpreter():
    from megakernels_amd.demos.latency.mk import LatencyMK_Interpreter
    from megakernels_amd.mk import DEFAULT_MK_DIR

    return LatencyMK_Interpreter(DEFAULT_MK_DIR), sys.modules["mk_llama"]


@pytest.fixture(scope="module")
def full_1b():
    from megakernels_amd.llama import LlamaConfig

    pair = make_model_pair(LlamaConfig.llama_1b(), max_len=16384 + 64)
    yield pair
    del pair
    torch.cuda.empty_cache()


@pytest.fixture(scope="module")
def full_8b():
    from megakernels_amd.llama import LlamaConfig

    pair = make_model_pair(LlamaConfig.llama_8b(), max_len=32768 + 64)
    yield pair
    del pair
    torch.cuda.empty_cache()


def _one_step(pair, pos, partitions):
    from oracle import pyvm

    model, model_gpu = pair
    cfg = model.config
    print(f"full-size step hidden={cfg.hidden_size} L={cfg.num_hidden_layers} inter={cfg.intermediate_size} "
          f"vocab={cfg.vocab_size} pos={pos} partitions={partitions}", flush=True)
    fill_kv_pair(model, model_gpu, upto=pos)
    schedule = build_schedule(model, 256, partitions=partitions)
    g = schedule.globs
    g.hidden_states.copy_(torch.randn(cfg.hidden_size, generator=torch.Generator().manual_seed(11)).to(torch.bfloat16))
    g.pos_id = pos
    _, schedule_gpu = mirror_to_gpu(model, schedule, model_gpu=model_gpu)
    print(f"  {len(schedule.get_linear_instructions())} instructions, {g.instructions.shape[1]} queue slots", flush=True)
    pyvm.interpret(g, schedule.get_linear_instructions())
    interp, mk_mod = _interpreter()
    interp.interpret(schedule_gpu.globs)
    mk_mod.check_status("cuda:0")
    # the caches are gigabytes: compare the row this step wrote and its neighbours
    rows = slice(max(pos - 1, 0), pos + 2)
    report = mismatches(g, schedule_gpu.globs, kv_rows=rows)
    assert not report, f"tensors differ from the checker: {report}"
    assert int(g.barriers.sum()) > 0
    return schedule, schedule_gpu


def _decode(pair, prefill, ntok, partitions):
    """`ntok` tokens in one launch through the fused loop, from the cache `_one_step` left."""
    from megakernels_amd.generators import MK_Generator
    from oracle import pyvm

    model, model_gpu = pair
    print(f"full-size decode prefill={prefill} ntok={ntok} partitions={partitions}", flush=True)
    schedule = build_schedule(model, 256, partitions=partitions)
    _, schedule_gpu = mirror_to_gpu(model, schedule, model_gpu=model_gpu)
    interp, mk_mod = _interpreter()
    tokens_cpu = torch.zeros(1, ntok + 1, dtype=torch.long)
    tokens_cpu[0, 0] = 4242
    pyvm.OracleGenerator(model, schedule).generate(tokens_cpu, prompt_len=prefill, ntok=ntok)
    tokens_gpu = tokens_cpu.to("cuda:0").clone()
    tokens_gpu[0, 1:] = 0
    MK_Generator(model_gpu, interp, schedule_gpu, fused_step=True, steps_per_launch=0).generate(
        tokens_gpu, prompt_len=prefill, ntok=ntok)
    mk_mod.check_status("cuda:0")
    assert tokens_gpu.cpu().tolist() == tokens_cpu.tolist()
    names = [n for n in schedule.globs.mutable_tensor_names() if n != "barriers"]
    report = mismatches(schedule.globs, schedule_gpu.globs, names=names, kv_rows=slice(prefill, prefill + ntok))
    assert not report, report


def test_c1_full_1b_short_context(full_1b):
    _one_step(full_1b, pos=40, partitions=1)
    _decode(full_1b, prefill=40, ntok=8, partitions=1)


def test_c2_full_1b_4096_positions_17_partitions(full_1b):
    _one_step(full_1b, pos=4100, partitions=17)
    _decode(full_1b, prefill=4100, ntok=8, partitions=17)


def test_c2_full_1b_64_steps_in_one_launch(full_1b):
    """The benchmark's own configuration held against the checker for a long launch: 64 decode steps
    at the full 1B shape, 4096+ cached positions, 17 partitions, without leaving the kernel.  Every
    step reads, with plain cached loads, K / V rows that earlier steps of the same launch wrote from
    other compute units, and every step starts behind a grid-wide hand-over of the previous token."""
    model, model_gpu = full_1b
    fill_kv_pair(model, model_gpu, upto=4100)
    _decode(full_1b, prefill=4100, ntok=64, partitions=17)


def test_c3_full_1b_16384_positions_24_partitions(full_1b):
    _one_step(full_1b, pos=16390, partitions=24)
    _decode(full_1b, prefill=16390, ntok=4, partitions=24)


def test_c4_full_8b_short_context(full_8b):
    schedule, _ = _one_step(full_8b, pos=40, partitions=1)
    cfg = full_8b[0].config
    assert cfg.intermediate_size // schedule.globs.matvec_reduction_size == 7   # the 4 + 2 + 1 partial-sum path
    _decode(full_8b, prefill=40, ntok=4, partitions=1)


def test_c5_full_8b_32768_positions_24_partitions(full_8b):
    schedule, _ = _one_step(full_8b, pos=32770, partitions=24)
    assert schedule.globs.instructions.shape[1] >= 150
    _decode(full_8b, prefill=32770, ntok=3, partitions=24)


def test_c5_full_8b_32768_positions_32_partitions_through_the_tree(full_8b):
    """the partition count the benchmark picks for this shape: one job per worker and KV head, merged by a
    two-level reduction tree; every partition streams 1024 positions through the double-buffered row stream"""
    _one_step(full_8b, pos=32770, partitions=32)
    _decode(full_8b, prefill=32770, ntok=2, partitions=32)

"""Instruction encoding and scheduling: pure integer logic, pinned against
(a) the reference's own scheduler output for Llama-3.2-1B on 132 and 148
workers (tests/golden/reference_schedules.json, written by
tests/golden/make_schedule_fixtures.py), (b) closed forms and coverage
invariants, and (c) the word layouts the reference's device parsers read."""

import json
from collections import Counter
from pathlib import Path

import pytest
import torch

from helpers import shape_only_model
from megakernels_amd.demos.latency.instructions import (
    AttentionReduction, DownProjResidual, LayerNorm_QKV_MatVecRopeAppend, LayerNormDoubleMatVecSiLU,
    O_ProjResidual, PartialAttention, RMS_LM_Head,
)
from megakernels_amd.demos.latency.scheduler import (
    LatencyScheduleBuilder, MAX_ATTENTION_PARTITIONS, pick_num_attention_partitions,
)
from megakernels_amd.instructions import Instruction, NoOp
from megakernels_amd.llama import LlamaConfig
from megakernels_amd.scheduler import (
    assign_to_sms, collect_into_waves, serialize_and_pad, tensorize_instructions,
)
from megakernels_amd.utils import set_sm_count_override

GOLDEN = json.loads((Path(__file__).parent / "golden" / "reference_schedules.json").read_text())


def build(cfg, workers, **kw):
    set_sm_count_override(workers)
    sched = LatencyScheduleBuilder.build(shape_only_model(cfg), **kw)
    sched.globs.pos_id = 40
    return sched


def cfg_1b(layers=2):
    return LlamaConfig(num_hidden_layers=layers)


# ---- (c) word layouts, as the reference's device code parses them -----------------------------


def test_word_layouts():
    # rms_matvec_rope_append.cu:38-41: [op, layer, start, end]
    assert LayerNorm_QKV_MatVecRopeAppend(3, 10, 12).serialize() == [1, 3, 10, 12]
    # attention_partial.cu:46-49: [op, layer, kv_head, num_partials, partial_idx]
    assert PartialAttention(2, 5, 7, 6).serialize() == [2, 2, 5, 7, 6]
    # attention_reduction.cu:34-45: [op, layer, head_start, num_partials, is_terminal, n, list..., out]
    assert AttentionReduction(1, 8, 3, True, [0, 1, 2], None).serialize() == [3, 1, 8, 3, 1, 3, 0, 1, 2, 0]
    assert AttentionReduction(1, 8, 3, False, [2, 1], 5).serialize() == [3, 1, 8, 3, 0, 2, 2, 1, 5]
    # matvec_adds.cu:26-34: [op, layer, start, end, reduction_block]
    assert O_ProjResidual(4, 7, 8, 0).serialize() == [4, 4, 7, 8, 0]
    assert DownProjResidual(4, 6, 8, 3).serialize() == [6, 4, 6, 8, 3]
    # upgate.cu:24-26: [op, layer, n, blocks...]
    assert LayerNormDoubleMatVecSiLU(9, [3, 135, 267]).serialize() == [5, 9, 3, 3, 135, 267]
    # rms_lm_head.cu:20-22: [op, start, end]
    assert RMS_LM_Head(100, 161).serialize() == [7, 100, 161]
    assert NoOp().serialize() == [0]
    assert serialize_and_pad(NoOp()) == [0] * 32
    assert len(serialize_and_pad(RMS_LM_Head(1, 2))) == 32


def test_words_round_trip():
    sched = build(cfg_1b(), 132, num_attention_partitions=5)
    for ins in sched.get_linear_instructions():
        words = serialize_and_pad(ins)
        assert Instruction.from_words(words).serialize() == ins.serialize()


def test_too_long_instruction_is_rejected():
    with pytest.raises(AssertionError):
        serialize_and_pad(LayerNormDoubleMatVecSiLU(0, list(range(30))))


# ---- (a) the reference's own output ----------------------------------------------------------------


@pytest.mark.parametrize("workers", [132, 148])
def test_linear_schedule_matches_reference(workers):
    sched = build(cfg_1b(), workers)
    ours = [ins.serialize() for ins in sched.get_linear_instructions()]
    assert ours == GOLDEN[str(workers)]["linear"]


@pytest.mark.parametrize("workers", [132, 148])
@pytest.mark.parametrize("mode", ["rr", "zz", "wave", "dag"])
def test_assignment_matches_reference(workers, mode):
    sched = build(cfg_1b(), workers)
    queues = assign_to_sms(mode, schedule=sched)
    ours = [[ins.serialize() for ins in q] for q in queues]
    assert ours == GOLDEN[str(workers)]["queues"][mode]


# ---- (b) closed forms and invariants -------------------------------------------------------------


@pytest.mark.parametrize("workers", [132, 148, 256])
def test_instruction_count_closed_form(workers):
    layers = 3
    sched = build(cfg_1b(layers), workers)
    assert len(sched.dag_nodes) == layers * (3 * workers + 136) + workers


@pytest.mark.parametrize("cfg,workers", [(cfg_1b(), 132), (cfg_1b(), 256), (LlamaConfig.llama_8b(), 256)])
def test_every_block_is_covered_exactly_once(cfg, workers):
    cfg.num_hidden_layers = 2
    sched = build(cfg, workers)
    g = sched.globs
    H, KVH, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    for layer in range(cfg.num_hidden_layers):
        ins_l = [i for i in sched.get_linear_instructions() if getattr(i, "layer_idx", None) == layer]
        qkv = Counter(b for i in ins_l if i.opcode() == 1 for b in i.block_indices())
        assert qkv == Counter(range((H + 2 * KVH) * D // 16))
        attn = Counter((i.kv_head_idx, i.partial_idx) for i in ins_l if i.opcode() == 2)
        assert attn == Counter((k, 0) for k in range(KVH))
        oproj = Counter((i.reduction_block_idx, b) for i in ins_l if i.opcode() == 4
                        for b in range(i.start_block_idx, i.end_block_idx))
        assert oproj == Counter((grp, b) for grp in range(g.o_proj_col_groups()) for b in range(cfg.hidden_size // 16))
        upgate = Counter(b for i in ins_l if i.opcode() == 5 for b in i.block_idxs)
        assert upgate == Counter(range(cfg.intermediate_size // 16))
        down = [(i.reduction_block_idx, b) for i in ins_l if i.opcode() == 6
                for b in range(i.start_block_idx, i.end_block_idx)]
        # group-major order: the order in which the bf16 partial sums are applied
        assert down == [(grp, b) for grp in range(g.down_proj_col_groups()) for b in range(cfg.hidden_size // 16)]
    lm = Counter(b for i in sched.get_linear_instructions() if i.opcode() == 7
                 for b in range(i.start_output_block_idx, i.end_output_block_idx))
    assert lm == Counter(range(cfg.vocab_size // 16))


def test_barrier_targets_reproduce_the_reference_constants():
    g = build(cfg_1b(), 132).globs
    # python_vm.py:110,132,176,255,283-290
    assert (g.down_proj_total_jobs(), g.o_proj_total_jobs(), g.up_gate_total_blocks(), g.qkv_blocks_per_head()) == (512, 128, 512, 4)
    g8 = build(LlamaConfig.llama_8b(), 256).globs
    assert (g8.o_proj_col_groups(), g8.down_proj_col_groups()) == (2, 7)
    assert g8.down_proj_total_jobs() == 7 * 256 and g8.o_proj_total_jobs() == 512 and g8.qkv_blocks_per_head() == 8


def test_qkv_ranges_use_round_half_even():
    # 192 blocks over 256 workers: b = 0.75; round(0.75 * 2) = round(1.5) = 2, round(0.75 * 6) = round(4.5) = 4
    sched = build(cfg_1b(1), 256)
    qkv = [i for i in sched.get_linear_instructions() if i.opcode() == 1]
    assert len(qkv) == 256
    assert [(i.start_output_block_idx, i.end_output_block_idx) for i in qkv[:7]] == [
        (0, 1), (1, 2), (2, 2), (2, 3), (3, 4), (4, 4), (4, 5)]
    assert sum(1 for i in qkv if i.start_output_block_idx == i.end_output_block_idx) == 64


def test_round_robin_queue_property_and_padding():
    sched = build(cfg_1b(), 132)
    linear = sched.get_linear_instructions()
    queues = assign_to_sms("rr", schedule=sched)
    for w, q in enumerate(queues):
        assert [i.serialize() for i in q] == [i.serialize() for i in linear[w::132]]
    tensorize_instructions(sched.globs, queues)
    ins = sched.globs.instructions
    longest = -(-len(linear) // 132)
    assert tuple(ins.shape) == (132, longest, 32) and ins.dtype == torch.int32
    assert tuple(sched.globs.timings.shape) == (132, longest, 128)
    short = len(linear) % 132
    assert bool((ins[short:, -1] == 0).all()) and bool((ins[:short, -1, 0] != 0).all())


@pytest.mark.parametrize("mode", ["zz", "wave", "dag"])
def test_other_policies_are_permutations(mode):
    sched = build(cfg_1b(), 256)
    queues = assign_to_sms(mode, schedule=sched)
    got = Counter(tuple(i.serialize()) for q in queues for i in q)
    want = Counter(tuple(i.serialize()) for i in sched.get_linear_instructions())
    assert got == want
    with pytest.raises(ValueError):
        assign_to_sms("nope", schedule=sched)


def test_collect_into_waves():
    sched = build(cfg_1b(1), 132)
    waves = collect_into_waves(sched.get_linear_instructions())
    assert [w[0].opcode() for w in waves] == [1, 2, 4, 5, 6, 7]


def test_stop_after_op_and_layer_limit():
    sched = build(cfg_1b(4), 132, stop_after_op="oproj", layer_limit=1)
    ops = {i.opcode() for i in sched.get_linear_instructions()}
    assert ops == {1, 2, 4}
    sched = build(cfg_1b(4), 132, layer_limit=2)
    assert 7 not in {i.opcode() for i in sched.get_linear_instructions()}


def test_split_kv_schedule():
    P = 6
    sched = build(cfg_1b(1), 256, num_attention_partitions=P)
    g = sched.globs
    assert not g.skip_attn_reduction
    ins = sched.get_linear_instructions()
    partials = [i for i in ins if i.opcode() == 2]
    assert [(i.kv_head_idx, i.num_partials, i.partial_idx) for i in partials] == [(k, P, p) for k in range(8) for p in range(P)]
    reds = [i for i in ins if i.opcode() == 3]
    assert [i.head_start_idx for i in reds] == list(range(0, 32, 4))
    assert all(i.is_terminal and i.reduction_list == list(range(P)) and i.num_partials == P for i in reds)
    # order: partials, then reductions, then O projection
    kinds = [i.opcode() for i in ins]
    assert kinds.index(3) > max(j for j, k in enumerate(kinds) if k == 2)
    assert kinds.index(4) > max(j for j, k in enumerate(kinds) if k == 3)
    with pytest.raises(AssertionError):
        build(cfg_1b(1), 256, num_attention_partitions=MAX_ATTENTION_PARTITIONS * MAX_ATTENTION_PARTITIONS + 1)
    with pytest.raises(AssertionError):          # 250 partitions + 10 first-level merges need 260 slots
        build(cfg_1b(1), 256, num_attention_partitions=250)
    assert pick_num_attention_partitions(4096, 64) == 17
    assert pick_num_attention_partitions(32, 128) == 1
    assert pick_num_attention_partitions(16384, 64) == 24
    set_sm_count_override(256)
    assert pick_num_attention_partitions(32768, 64, num_kv_heads=8, head_dim=128) == 32   # one per worker and KV head
    assert pick_num_attention_partitions(16384, 64, num_kv_heads=8, head_dim=64) == 24    # jobs too short for a tree
    assert pick_num_attention_partitions(16384, 64, num_kv_heads=8) == 24
    assert pick_num_attention_partitions(4096, 64, num_kv_heads=8, head_dim=64) == 17
    set_sm_count_override(132)
    assert pick_num_attention_partitions(32768, 64, num_kv_heads=8, head_dim=128) == 24


@pytest.mark.parametrize("P", [26, 32, 64])
def test_reduction_tree_schedule(P):
    """More partitions than one reduction can list: first-level merges over consecutive runs, written
    behind the partitions' slots, then one terminal merge over their outputs that waits for the
    partitions plus the first-level merges (the reference's open TODO, demos/latency/scheduler.py:21-35)."""
    from megakernels_amd.demos.latency.scheduler import reduction_tree_runs

    sched = build(cfg_1b(1), 256, num_attention_partitions=P)
    ins = sched.get_linear_instructions()
    runs = reduction_tree_runs(P)
    assert len(runs) == -(-P // MAX_ATTENTION_PARTITIONS) and runs[0][0] == 0 and runs[-1][1] == P
    assert all(a[1] == b[0] for a, b in zip(runs, runs[1:])) and max(hi - lo for lo, hi in runs) <= MAX_ATTENTION_PARTITIONS
    reds = [i for i in ins if i.opcode() == 3]
    assert len(reds) == 8 * (len(runs) + 1)
    for head_start in range(0, 32, 4):
        mine = [i for i in reds if i.head_start_idx == head_start]
        first, last = mine[:-1], mine[-1]
        assert [tuple(i.reduction_list[k] for k in (0, -1)) for i in first] == [(lo, hi - 1) for lo, hi in runs]
        assert all(not i.is_terminal and i.num_partials == P and i.output_partial_idx == P + k for k, i in enumerate(first))
        assert last.is_terminal and last.num_partials == P + len(runs) and last.reduction_list == [P + k for k in range(len(runs))]
    # every instruction still fits the 32-word format, and the DAG orders merges after what they read
    from megakernels_amd.scheduler import serialize_and_pad
    assert all(len(serialize_and_pad(i)) == 32 for i in reds)
    kinds = [i.opcode() for i in ins]
    assert kinds.index(4) > max(j for j, k in enumerate(kinds) if k == 3)


def test_complete_residual_sets_is_what_the_joint_flag_promises():
    """The launch shim sets MK_FLAG_JOINT_RESIDUAL only when every (projection, layer, row block) in the
    instruction tensor has the jobs of all its column groups, each once."""
    import importlib
    import sys

    from megakernels_amd.mk import DEFAULT_MK_DIR

    sys.path.append(str(DEFAULT_MK_DIR))
    shim = importlib.import_module("mk_llama")
    cfg = cfg_1b(2)
    for workers in (132, 256):
        sched = build(cfg, workers)
        queues = assign_to_sms("rr", schedule=sched)
        tensorize_instructions(sched.globs, queues)
        words = sched.globs.instructions
        assert shim.complete_residual_sets(words, 2048, 8192, 2048)
        # the cached answer goes when the tensor is written to: drop one down-projection job
        w, s = [(w, s) for w in range(words.shape[0]) for s in range(words.shape[1]) if words[w, s, 0] == 6][3]
        saved = words[w, s].clone()
        words[w, s] = 0
        assert not shim.complete_residual_sets(words, 2048, 8192, 2048)
        # the same job twice is not a complete set either
        words[w, s] = saved
        assert shim.complete_residual_sets(words, 2048, 8192, 2048)
        spare = [(w2, s2) for w2 in range(words.shape[0]) for s2 in range(words.shape[1]) if words[w2, s2, 0] == 0]
        if spare:
            words[spare[0]] = saved
            assert not shim.complete_residual_sets(words, 2048, 8192, 2048)
    # a single column group (O projection of the 1B shape) never needs the promise
    only_o = torch.zeros(4, 2, 32, dtype=torch.int32)
    only_o[0, 0, :5] = torch.tensor([4, 0, 0, 1, 0])
    assert shim.complete_residual_sets(only_o, 2048, 8192, 2048)


@pytest.mark.parametrize("mode", ["rr", "zz", "wave", "dag"])
def test_every_assignment_policy_lets_all_queues_finish(mode):
    """Queues run in order and wait on counters; the job of a residual projection's last column group
    also waits for the other groups' jobs of its rows when the jobs run on their own.  Every policy
    keeps the queues free of an instruction stuck behind one that waits for it."""
    from megakernels_amd.demos.latency.scheduler import check_queues_make_progress

    for cfg, workers, kw in ((cfg_1b(2), 132, {}), (cfg_1b(2), 256, {"num_attention_partitions": 5}),
                             (LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=2, num_attention_heads=32,
                                          num_key_value_heads=8, head_dim=128, vocab_size=4096), 256, {"num_attention_partitions": 30})):
        sched = build(cfg, workers, **kw)
        check_queues_make_progress(sched.globs, assign_to_sms(mode, schedule=sched))


def test_a_queue_order_that_cannot_finish_is_reported():
    from megakernels_amd.demos.latency.scheduler import check_queues_make_progress

    sched = build(cfg_1b(1), 64)
    queues = assign_to_sms("rr", schedule=sched)
    check_queues_make_progress(sched.globs, queues)
    # put the collecting job (last column group) of some rows in front of the job of another group
    # of the same rows, on one worker: it waits for a job that is queued behind it
    jobs = {}
    for w, q in enumerate(queues):
        for s, ins in enumerate(q):
            if isinstance(ins, DownProjResidual):
                jobs[(ins.start_block_idx, ins.reduction_block_idx)] = (w, s)
    block = next(b for (b, g) in jobs if g == 3 and (b, 0) in jobs)
    (wa, sa), (wb, sb) = jobs[(block, 3)], jobs[(block, 0)]
    collector, other = queues[wa][sa], queues[wb][sb]
    del queues[wb][sb]
    queues[wa].insert(sa + 1, other)
    with pytest.raises(AssertionError, match="can never finish"):
        check_queues_make_progress(sched.globs, queues)
    # an instruction in front of the producer of its own input: the same
    sched = build(cfg_1b(1), 64)
    queues = assign_to_sms("rr", schedule=sched)
    w = next(w for w, q in enumerate(queues) if any(isinstance(i, LayerNormDoubleMatVecSiLU) for i in q))
    s = next(s for s, i in enumerate(queues[w]) if isinstance(i, LayerNormDoubleMatVecSiLU))
    queues[w].insert(0, queues[w].pop(s))
    with pytest.raises(AssertionError, match="can never finish"):
        check_queues_make_progress(sched.globs, queues)

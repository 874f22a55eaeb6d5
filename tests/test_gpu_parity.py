"""GPU parity: the HIP megakernel, called through the C ABI of libmk_llama.so
(via the mk_llama shim), against the C restatement of the reference's Python
VM on identical seeded inputs.  The bar is BIT-EXACT equality of every buffer
the VM writes: hidden state, Q, KV rows, attention outputs and intermediates,
silu, logits, and the barrier counters."""

import pytest
import torch

from helpers import (
    build_schedule, config_1b_slice, config_8b_slice, config_tiny, fill_kv, make_model,
    mirror_to_gpu, mismatches,
)

pytestmark = pytest.mark.gpu


def _gpu_step(schedule_gpu):
    import sys
    from megakernels_amd.mk import DEFAULT_MK_DIR
    from megakernels_amd.demos.latency.mk import LatencyMK_Interpreter

    interp = LatencyMK_Interpreter(DEFAULT_MK_DIR)
    interp.interpret(schedule_gpu.globs)
    mk_mod = sys.modules["mk_llama"]
    mk_mod.check_status("cuda:0")


def _one_step_case(cfg, workers, pos, partitions=1, sched="rr", max_len=256, seed=0):
    from oracle import pyvm

    print(f"case hidden={cfg.hidden_size} D={cfg.head_dim} L={cfg.num_hidden_layers} workers={workers} "
          f"pos={pos} partitions={partitions} sched={sched}", flush=True)
    model = make_model(cfg, max_len=max_len, seed=seed)
    fill_kv(model, upto=pos)
    schedule = build_schedule(model, workers, partitions=partitions, sched=sched)
    g = schedule.globs
    gen = torch.Generator().manual_seed(11)
    g.hidden_states.copy_(torch.randn(cfg.hidden_size, generator=gen).to(torch.bfloat16))
    g.pos_id = pos
    model_gpu, schedule_gpu = mirror_to_gpu(model, schedule)
    pyvm.interpret(g, schedule.get_linear_instructions())
    _gpu_step(schedule_gpu)
    report = mismatches(g, schedule_gpu.globs)
    assert not report, f"tensors differ from the checker: {report}"


def test_tiny_single_partition():
    _one_step_case(config_tiny(), workers=16, pos=37)


def test_tiny_position_zero():
    _one_step_case(config_tiny(), workers=16, pos=0)


def test_tiny_split_kv():
    _one_step_case(config_tiny(), workers=16, pos=200, partitions=3)


def test_tiny_split_kv_with_empty_partition():
    # 2 KV blocks over 5 partitions: partitions 2..4 are empty (out 0, lse -inf)
    _one_step_case(config_tiny(), workers=16, pos=20, partitions=5)


def test_1b_slice_256_workers():
    _one_step_case(config_1b_slice(), workers=256, pos=150)


def test_1b_slice_reference_worker_counts():
    _one_step_case(config_1b_slice(layers=1), workers=132, pos=64)
    _one_step_case(config_1b_slice(layers=1), workers=148, pos=65)


def test_1b_slice_split_kv_long_context():
    _one_step_case(config_1b_slice(layers=1), workers=256, pos=4100, partitions=17, max_len=4352)


def test_1b_slice_other_assignments():
    for sched in ("zz", "wave", "dag"):
        _one_step_case(config_1b_slice(layers=1), workers=256, pos=33, sched=sched)


def test_8b_slice_column_groups():
    _one_step_case(config_8b_slice(), workers=256, pos=77)


def test_8b_slice_shared_qkv_blocks_under_every_assignment():
    """On the 4096-wide shape neighbouring workers whose QKV instructions of a layer differ by one block share
    the larger one's last block (rows 8-15 go to the neighbour).  Who neighbours whom depends on the assignment,
    and with fewer workers than instructions per layer a worker holds several QKV instructions (no sharing then):
    results and barrier counts are the checker's in every case."""
    for sched in ("rr", "zz", "wave", "dag"):
        _one_step_case(config_8b_slice(layers=2), workers=256, pos=33, sched=sched)
    _one_step_case(config_8b_slice(layers=2), workers=250, pos=33)   # 384 blocks over 250 workers: other pairings
    _one_step_case(config_8b_slice(layers=2), workers=100, pos=33)


def test_8b_slice_split_kv():
    _one_step_case(config_8b_slice(), workers=256, pos=1500, partitions=8, max_len=2048)


@pytest.mark.parametrize("shape", ["tiny", "1b", "8b"])
def test_column_group_jobs_alone_and_jointly(shape):
    """The residual projections' column-group jobs give the checker's bits both ways: each job on its
    own (partial sums handed to the last group's job) and, the default for complete schedules, jointly
    (the jobs of a block share its rows).  tiny: 2 down-projection groups; 1b: 4; 8b slice: 2
    O-projection groups run jointly, 3 down-projection groups cannot (3 does not divide 16)."""
    import sys
    from megakernels_amd.mk import get_mk_module

    mk_mod = get_mk_module()
    cfg, workers = {"tiny": (config_tiny(), 16), "1b": (config_1b_slice(), 256), "8b": (config_8b_slice(), 256)}[shape]
    try:
        for mode in (False, None):
            mk_mod.joint_residual_default = mode
            _one_step_case(cfg, workers=workers, pos=45)
    finally:
        mk_mod.joint_residual_default = None


def test_jobs_of_one_block_in_a_row_run_as_one():
    """A worker that holds several column-group jobs of the same blocks one after the other executes
    them in one go (pieces of 4, 2 or 1 jobs).  The 1B shape has 4 down-projection groups; the queues
    are rearranged so that workers hold groups (0, 1, 2, 3), (1, 2, 3), (2, 3), (0, 1) in a row, in
    falling order (1, 0) - which is no run - and single jobs.  Results and barrier counts are the checker's."""
    from megakernels_amd.demos.latency.instructions import DownProjResidual
    from megakernels_amd.scheduler import assign_to_sms, tensorize_instructions
    from oracle import pyvm

    cfg, workers, pos = config_1b_slice(), 256, 45
    print(f"case rearranged down-projection jobs hidden={cfg.hidden_size} workers={workers} pos={pos}", flush=True)
    model = make_model(cfg, max_len=256, seed=0)
    fill_kv(model, upto=pos)
    schedule = build_schedule(model, workers)
    g = schedule.globs
    queues = assign_to_sms("rr", schedule=schedule)
    for layer in range(cfg.num_hidden_layers):
        jobs = {}
        for queue in queues:
            for ins in [i for i in queue if isinstance(i, DownProjResidual) and i.layer_idx == layer]:
                jobs[(ins.start_block_idx, ins.end_block_idx, ins.reduction_block_idx)] = ins
                queue.remove(ins)
        ranges = sorted({key[:2] for key in jobs})
        assert all((*r, grp) in jobs for r in ranges for grp in range(4)), "complete sets of 4 column groups"
        patterns = [[(0, 1, 2, 3)], [(1, 2, 3), (0,)], [(1, 0), (2, 3)], [(0, 1), (3, 2)]]
        worker = 0
        for n, r in enumerate(ranges):
            for groups in patterns[n % 4]:
                # the layer's other instructions come first in every queue: down is a layer's last op
                at = max((k + 1 for k, i in enumerate(queues[worker]) if getattr(i, "layer_idx", -1) == layer), default=0)
                queues[worker][at:at] = [jobs[(*r, grp)] for grp in groups]
                worker = (worker + 1) % workers
    tensorize_instructions(g, queues)
    gen = torch.Generator().manual_seed(11)
    g.hidden_states.copy_(torch.randn(cfg.hidden_size, generator=gen).to(torch.bfloat16))
    g.pos_id = pos
    model_gpu, schedule_gpu = mirror_to_gpu(model, schedule)
    pyvm.interpret(g, schedule.get_linear_instructions())
    _gpu_step(schedule_gpu)
    report = mismatches(g, schedule_gpu.globs)
    assert not report, f"tensors differ from the checker: {report}"


def _suffix_case(cfg, workers, pos, start_after_op, partitions=1):
    """The reference's diff_test `start_after_op` (scripts/diff_test.py:122-152,198-208): the first part
    of a layer is run by the checker on both sets of buffers, the megakernel then gets only the
    instructions after it - its waits are satisfied by counts that were already in `barriers` when
    it started, its inputs were written by somebody else."""
    from megakernels_amd.scheduler import assign_to_sms, tensorize_instructions
    from oracle import pyvm

    print(f"suffix case hidden={cfg.hidden_size} workers={workers} pos={pos} start_after_op={start_after_op} "
          f"partitions={partitions}", flush=True)
    model = make_model(cfg)
    fill_kv(model, upto=pos)
    whole = build_schedule(model, workers, partitions=partitions, layer_limit=1)
    first = build_schedule(model, workers, partitions=partitions, layer_limit=1, stop_after_op=start_after_op)
    everything, head = whole.get_linear_instructions(), first.get_linear_instructions()
    assert 0 < len(head) < len(everything) and everything[: len(head)] == head
    tail = everything[len(head):]
    g = whole.globs
    g.hidden_states.copy_(torch.randn(cfg.hidden_size, generator=torch.Generator().manual_seed(13)).to(torch.bfloat16))
    g.pos_id = pos
    pyvm.interpret(g, head)
    tensorize_instructions(g, assign_to_sms("rr", instructions=tail, sm_count=workers))
    model_gpu, schedule_gpu = mirror_to_gpu(model, whole)
    assert int(schedule_gpu.globs.barriers.sum()) > 0
    pyvm.interpret(g, tail)
    _gpu_step(schedule_gpu)
    report = mismatches(g, schedule_gpu.globs)
    assert not report, f"tensors differ from the checker: {report}"


@pytest.mark.parametrize("start_after_op", ["qkv", "partial", "oproj", "upgate"])
def test_tiny_layer_started_after_an_op(start_after_op):
    _suffix_case(config_tiny(), workers=16, pos=21, start_after_op=start_after_op)


def test_tiny_split_kv_layer_started_after_the_reduction():
    _suffix_case(config_tiny(), workers=16, pos=44, start_after_op="reduction", partitions=3)


def test_tiny_split_kv_layer_started_after_the_partitions():
    # the partitions were counted in `barriers` before the launch: the reduction instructions do the
    # merging themselves although the schedule would let the last partition do it
    _suffix_case(config_tiny(), workers=16, pos=44, start_after_op="partial", partitions=3)


def test_1b_slice_layer_started_after_the_o_projection():
    _suffix_case(config_1b_slice(layers=2), workers=256, pos=70, start_after_op="oproj")


def _tiny_long_context(positions=8192):
    cfg = config_tiny()
    cfg.max_position_embeddings = positions      # length of the rotary tables
    return cfg


def test_tiny_partition_of_exactly_the_on_chip_limit():
    """One partition over 4096 cached positions fills the score buffer to the last slot."""
    _one_step_case(_tiny_long_context(), workers=16, pos=4095, max_len=4096 + 8)


def test_single_partition_beyond_the_score_buffer():
    """The reference's own schedule has one partition per KV head whatever the context length
    (demos/latency/scheduler.py:276-277, max_len_override=16384 in scripts/generate.py:43) and its
    kernel walks it block by block (attention_partial.cu:463-520).  Here a partition of more than 4096
    positions does not fit the on-chip score buffer and takes the path that recomputes the scores in
    its second pass: same bits."""
    _one_step_case(_tiny_long_context(), workers=16, pos=4100, max_len=4096 + 64)
    _one_step_case(_tiny_long_context(16448), workers=16, pos=16384, max_len=16384 + 64)


@pytest.mark.parametrize("pos", [255, 256, 257, 319, 511, 512, 513, 767, 768, 1023, 1024, 1025, 1300])
def test_tiny_row_stream_boundaries(pos):
    """Partitions around the edges of the double-buffered row stream (head_dim 64: the first 256 positions
    of a partition are requested ahead of the dependency, the rest streams in batches of 256): the newest
    position first, last or alone in a batch, a batch that ends with the partition, one position beyond."""
    _one_step_case(_tiny_long_context(2048), workers=16, pos=pos, max_len=1408)
    _one_step_case(_tiny_long_context(2048), workers=16, pos=pos, partitions=2, max_len=1408)


def test_8b_slice_row_stream_boundaries():
    # head_dim 128: 128 positions ahead of the dependency, batches of 128
    for pos in (127, 128, 129, 255, 256, 257, 400):
        _one_step_case(config_8b_slice(), workers=256, pos=pos, partitions=1, max_len=512)


def test_1b_slice_single_partition_long_context():
    _one_step_case(config_1b_slice(layers=1), workers=256, pos=5000, partitions=1, max_len=5120)


def test_8b_slice_long_partitions():
    # head_dim 128: two partitions of 3008 and 2993 positions (deep batches), then one of 6001 (recomputed)
    _one_step_case(config_8b_slice(), workers=256, pos=6000, partitions=2, max_len=6144)
    _one_step_case(config_8b_slice(), workers=256, pos=6000, partitions=1, max_len=6144)


def test_reduction_tree():
    """More partitions than one merge can list (25): first-level merges, then the terminal one."""
    _one_step_case(config_tiny(), workers=64, pos=600, partitions=32, max_len=1024)
    # 65 KV blocks over 64 partitions of two blocks: partitions 33..63 are empty, and so is the whole
    # last run of first-level merges
    _one_step_case(_tiny_long_context(), workers=96, pos=1029, partitions=64, max_len=1100)
    _one_step_case(config_1b_slice(layers=2), workers=256, pos=3000, partitions=40, max_len=3072)


def test_queue_longer_than_the_on_chip_window():
    """20 layers on 4 workers: 260 instructions per worker go through the 192-slot window in two
    fetches (the reference streams instructions from global memory, include/controller/instruction_fetch.cuh:10-27)."""
    import sys

    cfg = config_tiny(layers=20)
    _one_step_case(cfg, workers=4, pos=33, partitions=2)

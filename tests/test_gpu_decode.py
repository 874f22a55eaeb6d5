"""GPU: multi-step greedy decoding through the reference-shaped generator loop
(embedding, barrier reset, megakernel, argmax) must produce the checker's token
ids bit for bit and leave the same KV cache behind; plus the behaviour of the
launch boundary when things go wrong (every kernel still exits normally)."""

import ctypes
import sys

import pytest
import torch

from helpers import (
    build_schedule, config_1b_slice, config_8b_slice, config_tiny, fill_kv, make_model, mirror_to_gpu, mismatches,
)

pytestmark = pytest.mark.gpu


def _interpreter():
    from megakernels_amd.demos.latency.mk import LatencyMK_Interpreter
    return LatencyMK_Interpreter(), sys.modules["mk_llama"]


def _decode_case(cfg, workers, prefill, ntok, partitions=1, max_len=256, sched="rr", fused=False, steps_per_launch=1,
                 model=None):
    from megakernels_amd.generators import MK_Generator
    from oracle import pyvm

    print(f"decode case hidden={cfg.hidden_size} workers={workers} prefill={prefill} ntok={ntok} "
          f"partitions={partitions}", flush=True)
    if model is None:
        model = make_model(cfg, max_len=max_len)
    fill_kv(model, upto=prefill)
    schedule = build_schedule(model, workers, partitions=partitions, sched=sched)
    model_gpu, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, mk_mod = _interpreter()

    tokens_cpu = torch.zeros(1, ntok + 1, dtype=torch.long)
    tokens_cpu[0, 0] = 5
    pyvm.OracleGenerator(model, schedule).generate(tokens_cpu, prompt_len=prefill, ntok=ntok)

    tokens_gpu = torch.zeros(1, ntok + 1, dtype=torch.long, device="cuda:0")
    tokens_gpu[0, 0] = 5
    gen = MK_Generator(model_gpu, interp, schedule_gpu, fused_step=fused, steps_per_launch=steps_per_launch)
    assert gen.fused_step == fused and gen.steps_per_launch == steps_per_launch
    gen.generate(tokens_gpu, prompt_len=prefill, ntok=ntok)
    mk_mod.check_status("cuda:0")
    assert tokens_gpu.cpu().tolist() == tokens_cpu.tolist()
    rows = slice(prefill, prefill + ntok)
    names = list(schedule.globs.mutable_tensor_names())
    if fused:
        # one launch per token: embedding, argmax and barrier reset happen inside it, so the
        # barriers end up zeroed instead of holding the last step's counts
        names.remove("barriers")
        assert int(schedule_gpu.globs.barriers.abs().sum()) == 0
    report = mismatches(schedule.globs, schedule_gpu.globs, names=names, kv_rows=rows)
    assert not report, report


def test_decode_tiny():
    _decode_case(config_tiny(), workers=16, prefill=20, ntok=12)


def test_decode_tiny_one_launch_per_token():
    _decode_case(config_tiny(), workers=16, prefill=20, ntok=12, fused=True)


def test_decode_tiny_one_launch_per_token_split_kv():
    _decode_case(config_tiny(), workers=16, prefill=30, ntok=20, partitions=3, fused=True)


def test_decode_1b_slice_one_launch_per_token():
    _decode_case(config_1b_slice(layers=3), workers=256, prefill=100, ntok=8, fused=True)


def test_decode_1b_slice_many_steps_split_kv_one_launch_per_token():
    # 160 consecutive launches, every one checked through its token: a race between workgroups would
    # have many chances to show
    _decode_case(config_1b_slice(layers=2), workers=256, prefill=500, ntok=160, partitions=3, max_len=1024, fused=True)


def test_decode_tiny_all_steps_in_one_launch():
    _decode_case(config_tiny(), workers=16, prefill=20, ntok=12, fused=True, steps_per_launch=0)


def test_decode_tiny_split_kv_seven_steps_per_launch():
    # launches of 7, 7 and 6 steps; positions 30..49 cross the 16-token block boundaries at 32 and 48
    _decode_case(config_tiny(), workers=16, prefill=30, ntok=20, partitions=3, fused=True, steps_per_launch=7)


def test_decode_1b_slice_all_steps_in_one_launch():
    _decode_case(config_1b_slice(layers=3), workers=256, prefill=100, ntok=8, fused=True, steps_per_launch=0)


def test_decode_1b_slice_many_steps_split_kv_in_one_launch():
    # 160 steps without leaving the kernel: every step's token is checked, and every step starts
    # behind a grid-wide hand-over of the previous token
    _decode_case(config_1b_slice(layers=2), workers=256, prefill=500, ntok=160, partitions=3, max_len=1024, fused=True,
                 steps_per_launch=0)


def test_decode_tiny_long_queue_and_reduction_tree_in_one_launch():
    # 213 slots per worker (two windows, refetched every step) and a two-level reduction tree
    _decode_case(config_tiny(layers=17), workers=4, prefill=20, ntok=6, partitions=2, fused=True, steps_per_launch=0)
    _decode_case(config_tiny(), workers=48, prefill=500, ntok=6, partitions=30, max_len=1024, fused=True, steps_per_launch=0)


def test_decode_8b_slice_all_steps_in_one_launch():
    _decode_case(config_8b_slice(layers=2), workers=256, prefill=50, ntok=4, partitions=2, fused=True, steps_per_launch=0)


def test_prefill_on_the_gpu_hands_its_cache_to_the_megakernel():
    """The reference's flow (scripts/generate.py:125-137): the prompt goes through the plain PyTorch
    forward on the GPU, which fills the KV cache and yields the first token; the megakernel decodes
    from there.  The checker starts from a copy of the cache the GPU prefill left, and must see the
    same tokens and the same appended KV rows."""
    from megakernels_amd.generators import MK_Generator
    from megakernels_amd.model_types import BatchState
    from oracle import pyvm

    cfg = config_1b_slice(layers=3)
    model = make_model(cfg, max_len=128)
    model_gpu = model.to("cuda:0")
    prompt = torch.randint(0, cfg.vocab_size, (1, 32), generator=torch.Generator().manual_seed(1))
    out = model_gpu(BatchState(input_ids=prompt.to("cuda:0"), position_ids=torch.arange(32, device="cuda:0")))
    first_token = int(out.output_ids[0, -1])
    for dst, src in zip(model.stacked_kv_cache, model_gpu.stacked_kv_cache):
        dst.copy_(src)
    assert float(model.stacked_kv_cache[0][:, :, :32].float().abs().sum()) > 0 and float(model.stacked_kv_cache[0][:, :, 32:].float().abs().sum()) == 0
    # the GPU prefill agrees with the CPU forward to bf16 rounding (different GEMM kernels, same maths)
    model_ref = make_model(cfg, max_len=128)
    model_ref(BatchState(input_ids=prompt, position_ids=torch.arange(32)))
    k_gpu, k_cpu = model.stacked_kv_cache[0][:, :, :32].float(), model_ref.stacked_kv_cache[0][:, :, :32].float()
    assert float((k_gpu - k_cpu).abs().max()) <= 2e-2 * float(k_cpu.abs().max())

    ntok = 8
    schedule = build_schedule(model, 256)
    _, schedule_gpu = mirror_to_gpu(model, schedule, model_gpu=model_gpu)
    interp, mk_mod = _interpreter()
    tokens_cpu = torch.zeros(1, ntok + 1, dtype=torch.long)
    tokens_cpu[0, 0] = first_token
    pyvm.OracleGenerator(model, schedule).generate(tokens_cpu, prompt_len=32, ntok=ntok)
    tokens_gpu = torch.zeros(1, ntok + 1, dtype=torch.long, device="cuda:0")
    tokens_gpu[0, 0] = first_token
    MK_Generator(model_gpu, interp, schedule_gpu, fused_step=True, steps_per_launch=0).generate(
        tokens_gpu, prompt_len=32, ntok=ntok, check=True)
    assert tokens_gpu.cpu().tolist() == tokens_cpu.tolist()
    names = [n for n in schedule.globs.mutable_tensor_names() if n != "barriers"]
    report = mismatches(schedule.globs, schedule_gpu.globs, names=names, kv_rows=slice(0, 32 + ntok))
    assert not report, report


def test_decode_from_a_hugging_face_checkpoint(tmp_path):
    """The whole user path: a checkpoint directory written by the installed third-party `transformers`
    (untied head, llama3 rope scaling), loaded with `from_pretrained`, decoded through the megakernel,
    token-exact against the checker."""
    transformers = pytest.importorskip("transformers")
    from megakernels_amd.llama import LlamaForCausalLM
    from megakernels_amd.model_types import ExtraModelConfig

    hf_cfg = transformers.LlamaConfig(
        vocab_size=1024, hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=8,
        num_key_value_heads=2, head_dim=64, max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=500000.0,
        tie_word_embeddings=False, attention_bias=False, mlp_bias=False,
        rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                      "original_max_position_embeddings": 64})
    torch.manual_seed(17)
    transformers.LlamaForCausalLM(hf_cfg).eval().save_pretrained(tmp_path, safe_serialization=True)
    model = LlamaForCausalLM.from_pretrained(tmp_path, ExtraModelConfig(interleave_rope=True, max_len_override=128))
    _decode_case(model.config, workers=16, prefill=24, ntok=10, partitions=2, fused=True, steps_per_launch=0, model=model)


def test_steps_past_the_kv_cache_are_refused():
    from megakernels_amd.generators import MK_Generator

    cfg = config_tiny()
    model = make_model(cfg, max_len=32)
    fill_kv(model, upto=8)
    schedule = build_schedule(model, 16)
    model_gpu, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, _ = _interpreter()
    tokens = torch.zeros(1, 64, dtype=torch.long, device="cuda:0")
    with pytest.raises(RuntimeError, match="run past the KV cache"):
        MK_Generator(model_gpu, interp, schedule_gpu, fused_step=True).generate(tokens, prompt_len=8, ntok=40)


def test_token_outside_the_vocabulary_is_reported():
    from megakernels_amd.generators import MK_Generator

    cfg = config_tiny()
    model = make_model(cfg, max_len=64)
    fill_kv(model, upto=8)
    schedule = build_schedule(model, 16)
    model_gpu, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, mk_mod = _interpreter()
    tokens = torch.zeros(1, 3, dtype=torch.long, device="cuda:0")
    tokens[0, 0] = cfg.vocab_size + 7
    MK_Generator(model_gpu, interp, schedule_gpu, fused_step=True).generate(tokens, prompt_len=8, ntok=1)
    code, *_ = mk_mod.read_status("cuda:0")
    assert code == 5


def test_decode_tiny_split_kv_crossing_block_boundaries():
    # positions 30..49 cross the 16-token block boundaries at 32 and 48
    _decode_case(config_tiny(), workers=16, prefill=30, ntok=20, partitions=3)


def test_decode_1b_slice():
    _decode_case(config_1b_slice(layers=3), workers=256, prefill=100, ntok=8)


def test_decode_1b_slice_long_context_split_kv():
    _decode_case(config_1b_slice(layers=2), workers=256, prefill=2000, ntok=6, partitions=9, max_len=2048 + 64)


def test_decode_8b_slice():
    _decode_case(config_8b_slice(layers=2), workers=256, prefill=50, ntok=4, partitions=2)


def test_hardware_bf16_conversion_equals_portable_formula():
    _, mk_mod = _interpreter()
    lib = mk_mod.load_library()
    lib.mk_llama_selftest_bf16.argtypes = [ctypes.POINTER(ctypes.c_uint64)]
    out = ctypes.c_uint64(123)
    assert lib.mk_llama_selftest_bf16(ctypes.byref(out)) == 0
    assert out.value == 0


def test_timings_are_recorded_on_request():
    model = make_model(config_tiny())
    fill_kv(model, upto=9)
    schedule = build_schedule(model, 16)
    schedule.globs.pos_id = 9
    _, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, mk_mod = _interpreter()
    g = schedule_gpu.globs
    interp.interpret(g)
    mk_mod.check_status("cuda:0")
    assert int(g.timings.abs().sum()) == 0          # off by default, like the reference build
    mk_mod.record_timings = True
    try:
        g.barriers.zero_()
        interp.interpret(g)
        mk_mod.check_status("cuda:0")
    finally:
        mk_mod.record_timings = False
    t = g.timings.cpu()
    ins = g.instructions.cpu()
    real = ins[:, :, 0] != 0
    from megakernels_amd.scripts import timeline as tl

    assert torch.equal(t[:, :, tl.OPCODE][real], ins[:, :, 0][real])    # opcode echoed
    # the records are the low 32 bits of one device-wide clock: start <= dependency seen <= input
    # ready <= rows done <= end for every instruction, and nothing took longer than a second
    ticks = t.to(torch.int64)

    def ordered(earlier, later, where):
        gap = (ticks[:, :, later] - ticks[:, :, earlier])[where] % (1 << 32)
        assert bool((gap < 100_000_000).all()), (earlier, later)

    for earlier, later in ((0, 1), (1, 2), (2, 3), (3, 4)):
        ordered(earlier, later, real)
    # the waves that do the work stamp the reference's own event slots (include/util.cuh:215-246):
    # measured, in order, for every matvec instruction that had rows
    matvec = real & (ins[:, :, 0] != 2) & (ins[:, :, 0] != 3) & (t[:, :, tl.FIRST_USE] != 0)
    assert int(matvec.sum()) > 0
    chain = (tl.START, tl.AT_GMEM_WAIT, tl.DONE_GMEM_WAIT, tl.LAUNCHER_START, tl.FIRST_USE, tl.LAST_USE,
             tl.AT_GMEM_STORE, tl.END)
    for earlier, later in zip(chain, chain[1:]):
        ordered(earlier, later, matvec)
    ordered(tl.FIRST_LOAD, tl.LAST_LOAD, matvec)
    ordered(tl.LAST_LOAD, tl.LAST_USE, matvec)
    signalling = matvec & (ins[:, :, 0] != 7)   # the LM head signals nobody inside the launch
    for earlier, later in ((tl.AT_GMEM_STORE, tl.DONE_GMEM_STORE), (tl.DONE_GMEM_STORE, tl.OUTPUT_READY),
                           (tl.OUTPUT_READY, tl.END)):
        ordered(earlier, later, signalling)
    assert torch.equal(t[:, :, tl.DONE_GMEM_WAIT][matvec], t[:, :, tl.DEP_READY][matvec])
    # attention and merge: the working waves stamp first use, stores and signal
    for op in (2, 3):
        sel = real & (ins[:, :, 0] == op)
        if int(sel.sum()):
            for earlier, later in ((tl.START, tl.AT_GMEM_STORE), (tl.AT_GMEM_STORE, tl.DONE_GMEM_STORE),
                                   (tl.DONE_GMEM_STORE, tl.OUTPUT_READY)):
                ordered(earlier, later, sel)
            # (in attention the storing waves signal on their own, after the controller wave has moved
            # on: its END can precede OUTPUT_READY; a merge leaves together, after the signal)
            if op == 3:
                ordered(tl.OUTPUT_READY, tl.END, sel)
    # one clock for all workers: the whole launch spans well under a second
    starts = ticks[:, :, 0][real]
    assert int(((starts - starts.min()) % (1 << 32)).max()) < 100_000_000


def test_unsatisfiable_dependency_times_out_and_reports():
    """A schedule whose attention never runs: the O projection's wait can never be satisfied.  With
    a short spin limit the workers give up, record the status and exit; nothing hangs."""
    model = make_model(config_tiny())
    fill_kv(model, upto=9)
    schedule = build_schedule(model, 16)
    g = schedule.globs
    g.pos_id = 9
    g.instructions[g.instructions[:, :, 0] == 2] = 0   # drop every attention instruction
    _, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, mk_mod = _interpreter()
    mk_mod.spin_limit_us = 20000
    try:
        interp.interpret(schedule_gpu.globs)
        code, worker, slot, opcode = mk_mod.read_status("cuda:0")
    finally:
        mk_mod.spin_limit_us = 0
    assert code == 1 and opcode == 4
    with pytest.raises(RuntimeError, match="timed out"):
        mk_mod.spin_limit_us = 20000
        try:
            schedule_gpu.globs.barriers.zero_()
            interp.interpret(schedule_gpu.globs)
            mk_mod.check_status("cuda:0")
        finally:
            mk_mod.spin_limit_us = 0
    # the workspace was cleaned: a valid schedule runs right after
    test_decode_tiny()


def test_missing_attention_partials_time_out_in_the_merge():
    """Split-KV schedule without its attention instructions: the merge waits for partition counters
    that never move, gives up at the spin limit and the whole grid drains."""
    model = make_model(config_tiny())
    fill_kv(model, upto=40)
    schedule = build_schedule(model, 16, partitions=2)
    g = schedule.globs
    g.pos_id = 40
    g.instructions[g.instructions[:, :, 0] == 2] = 0
    _, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, mk_mod = _interpreter()
    mk_mod.spin_limit_us = 20000
    try:
        interp.interpret(schedule_gpu.globs)
        code, worker, slot, opcode = mk_mod.read_status("cuda:0")
    finally:
        mk_mod.spin_limit_us = 0
    assert code == 1 and opcode in (3, 4)
    test_decode_tiny_split_kv_crossing_block_boundaries()


def test_failure_in_a_launch_of_several_steps_drains_the_grid():
    """The same broken schedule inside a launch of four steps: the workers that give up never reach the
    end of the step, the others find the failure while waiting for the step to be published, and no
    second step starts."""
    from megakernels_amd.generators import MK_Generator

    model = make_model(config_tiny())
    fill_kv(model, upto=40)
    schedule = build_schedule(model, 16, partitions=2)
    g = schedule.globs
    g.instructions[g.instructions[:, :, 0] == 2] = 0
    model_gpu, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, mk_mod = _interpreter()
    tokens = torch.full((1, 5), -1, dtype=torch.long, device="cuda:0")
    tokens[0, 0] = 5
    mk_mod.spin_limit_us = 20000
    try:
        MK_Generator(model_gpu, interp, schedule_gpu, fused_step=True, steps_per_launch=0).generate(tokens, prompt_len=40, ntok=4)
        code, worker, slot, opcode = mk_mod.read_status("cuda:0")
    finally:
        mk_mod.spin_limit_us = 0
    assert code == 1 and opcode in (3, 4)
    assert tokens[0, 2:].tolist() == [-1, -1, -1]      # nothing after the first step was produced
    test_decode_tiny_all_steps_in_one_launch()


def test_generator_raises_when_a_chunk_gave_up():
    """generate_with_eos looks at the kernel's status after every chunk, and generate(check=True) at
    its end: tokens of a launch that gave up are never handed on as text."""
    from megakernels_amd.generators import MK_Generator

    model = make_model(config_tiny())
    fill_kv(model, upto=12)
    schedule = build_schedule(model, 16)
    model_gpu, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, mk_mod = _interpreter()
    gen = MK_Generator(model_gpu, interp, schedule_gpu, fused_step=True, steps_per_launch=0)
    tokens = torch.zeros(1, 9, dtype=torch.long, device="cuda:0")
    tokens[0, 0] = 7
    schedule_gpu.globs.instructions[5, 1, 0] = 77      # an opcode the kernel does not know
    mk_mod.spin_limit_us = 20000
    try:
        with pytest.raises(RuntimeError, match="unknown opcode"):
            gen.generate_with_eos(tokens, prompt_len=12, ntok=9, eos_token_check_interval=4, eos_token_ids=[1023])
        with pytest.raises(RuntimeError, match="unknown opcode"):
            gen.generate(tokens, prompt_len=12, ntok=4, check=True)
    finally:
        mk_mod.spin_limit_us = 0
    # the failed launches left nothing behind: the repaired schedule decodes
    schedule_gpu.globs.instructions.copy_(schedule.globs.instructions)
    gen.generate(tokens, prompt_len=12, ntok=4, check=True)


def test_unknown_opcode_and_bad_fields_are_reported():
    model = make_model(config_tiny())
    schedule = build_schedule(model, 16)
    g = schedule.globs
    g.pos_id = 3
    _, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, mk_mod = _interpreter()
    gg = schedule_gpu.globs
    good = gg.instructions.clone()
    mk_mod.spin_limit_us = 20000
    try:
        gg.instructions[3, 0, 0] = 42
        interp.interpret(gg)
        code, worker, slot, opcode = mk_mod.read_status("cuda:0")
        assert (code, worker, slot, opcode) == (2, 3, 0, 42)
        gg.instructions.copy_(good)
        gg.instructions[2, 0, 1] = 99                  # layer index out of range
        gg.barriers.zero_()
        interp.interpret(gg)
        assert mk_mod.read_status("cuda:0")[0] == 4
    finally:
        mk_mod.spin_limit_us = 0


def test_launch_argument_validation():
    model = make_model(config_tiny())
    schedule = build_schedule(model, 16)
    _, schedule_gpu = mirror_to_gpu(model, schedule)
    interp, mk_mod = _interpreter()
    gg = schedule_gpu.globs
    gg.pos_id = 10_000_000
    with pytest.raises(RuntimeError, match="pos_id"):
        interp.interpret(gg)
    gg.pos_id = 1
    saved = gg.logits
    gg.logits = torch.zeros(7, dtype=torch.bfloat16, device="cuda:0")
    with pytest.raises(RuntimeError, match="logits"):
        interp.interpret(gg)
    gg.logits = saved
    saved = gg.instructions
    gg.instructions = saved[:, :, :16].contiguous()
    with pytest.raises(RuntimeError, match="instructions"):
        interp.interpret(gg)
    gg.instructions = saved


def test_diff_test_outfile_dump(tmp_path):
    """tests/diff_test.py outfile=: the dump the reference's timing tools read
    (scripts/diff_test.py:231-242) - keys, shapes, and measured events in the reference's slots
    (include/util.cuh:215-246) in order for the instructions that ran."""
    import pickle
    from pathlib import Path

    sys.path.insert(0, str(Path(__file__).resolve().parent))
    import diff_test
    from megakernels_amd.scripts import timeline as tl

    out = tmp_path / "timings.pkl"
    diff_test.main(diff_test.parse(["model=tiny", "prompt_len=20", "ntok=5", "num_attention_partitions=3", f"outfile={out}"]))
    with open(out, "rb") as f:
        data = pickle.load(f)   # written a moment ago by this test
    assert set(data) == {"timings", "timings_native", "instructions", "python_instructions", "cost_per_sm"}
    workers, slots = data["instructions"].shape[:2]
    assert workers == 16 and tuple(data["instructions"].shape) == (workers, slots, 32)
    assert tuple(data["timings"].shape) == (workers, slots, 128) == tuple(data["timings_native"].shape)
    assert len(data["python_instructions"]) == workers and len(data["cost_per_sm"]) == workers
    assert all(len(q) <= slots for q in data["python_instructions"])
    assert all(cost > 0 for cost in data["cost_per_sm"])
    t = data["timings"].to(torch.int64)
    ins = data["instructions"]
    real = ins[:, :, 0] != 0
    assert int(real.sum()) > 0 and int(t[~real].abs().sum()) == 0
    # ticks since the launch's first instruction: somebody starts at zero, nothing lasts a second
    assert int(t[:, :, tl.START][real].min()) == 0 and int(t[real].max()) < 100_000_000
    assert torch.equal(t[:, :, tl.OPCODE][real], ins[:, :, 0][real].to(torch.int64))
    matvec = real & (ins[:, :, 0] != 2) & (ins[:, :, 0] != 3) & (t[:, :, tl.FIRST_USE] != 0)
    assert int(matvec.sum()) > 0
    chain = (tl.START, tl.AT_GMEM_WAIT, tl.DONE_GMEM_WAIT, tl.LAUNCHER_START, tl.FIRST_USE, tl.LAST_USE, tl.AT_GMEM_STORE, tl.END)
    for earlier, later in zip(chain, chain[1:]):
        assert bool((t[:, :, earlier][matvec] <= t[:, :, later][matvec]).all()), (earlier, later)
    # the stages only the reference has are over when an instruction starts
    for stage in tl.REFERENCE_ONLY_STAGES:
        assert torch.equal(t[:, :, stage][real], t[:, :, tl.START][real])

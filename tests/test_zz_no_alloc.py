"""mk_llama_launch_static - the launch that allocates nothing and keeps its workspace in an array
inside the library - against mk_llama_launch on the same inputs: every buffer the kernel writes
must come out bit for bit the same.  Two calls in a row share the array, the second with smaller
shapes (its counters lie where the first call left residual partial sums), then a third, larger
again, after a launch that gave up and left its status in the array."""

import sys

import pytest
import torch

from helpers import build_schedule, config_1b_slice, config_8b_slice, config_tiny, fill_kv, make_model, mirror_to_gpu, mismatches

pytestmark = pytest.mark.gpu


def _interpreter():
    from megakernels_amd.demos.latency.mk import LatencyMK_Interpreter
    from megakernels_amd.mk import DEFAULT_MK_DIR

    interp = LatencyMK_Interpreter(DEFAULT_MK_DIR)
    return interp, sys.modules["mk_llama"]


def _both_ways(cfg, workers, pos, partitions, max_len=256):
    """One decode step through each entry point from identical inputs; returns the two buffer bundles."""
    print(f"case hidden={cfg.hidden_size} L={cfg.num_hidden_layers} workers={workers} pos={pos} partitions={partitions}", flush=True)
    interp, mk_mod = _interpreter()
    model = make_model(cfg, max_len=max_len)
    fill_kv(model, upto=pos)
    schedule = build_schedule(model, workers, partitions=partitions)
    g = schedule.globs
    g.hidden_states.copy_(torch.randn(cfg.hidden_size, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16))
    g.pos_id = pos
    _, plain = mirror_to_gpu(model, schedule)
    _, static = mirror_to_gpu(model, schedule)
    interp.interpret(plain.globs)
    mk_mod.check_status("cuda:0")
    # what the instruction tensor promises is looked up once per tensor (a copy to the host): before the
    # launch that must not allocate
    mk_mod.complete_residual_sets(static.globs.instructions, cfg.hidden_size, cfg.intermediate_size, min(2048, cfg.hidden_size))
    import gc

    gc.collect()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before, _ = torch.cuda.mem_get_info()     # the driver's own count: sees a hipMalloc inside the library too
    mk_mod.static_scratch = True
    try:
        interp.interpret(static.globs)
        mk_mod.check_status("cuda:0")
    finally:
        mk_mod.static_scratch = False
    free_after, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_allocated() <= before, "the static launch allocated device memory through torch"
    assert free_after >= free_before, f"the static launch took {free_before - free_after} bytes of device memory from the driver"
    return plain.globs, static.globs


def test_static_scratch_launch_matches_the_ordinary_launch_on_consecutive_calls():
    # an 8B-shaped slice first: 3 down-projection groups of 4096 partial sums in the workspace
    a, b = _both_ways(config_8b_slice(), workers=256, pos=300, partitions=3, max_len=512)
    assert not mismatches(a, b), mismatches(a, b)
    assert int(b.barriers.sum()) > 0
    # then the smallest shape: its whole workspace lies inside what the first call used
    a, b = _both_ways(config_tiny(), workers=16, pos=37, partitions=2)
    assert not mismatches(a, b), mismatches(a, b)
    a, b = _both_ways(config_1b_slice(layers=2), workers=256, pos=150, partitions=1)
    assert not mismatches(a, b), mismatches(a, b)


def test_static_scratch_recovers_after_a_launch_that_gave_up():
    interp, mk_mod = _interpreter()
    cfg = config_tiny()
    model = make_model(cfg, max_len=128)
    fill_kv(model, upto=20)
    schedule = build_schedule(model, 16)
    schedule.globs.pos_id = 20
    _, broken = mirror_to_gpu(model, schedule)
    broken.globs.instructions[3, 0, 0] = 99          # unknown opcode: the launch records a status and drains
    mk_mod.static_scratch = True
    mk_mod.spin_limit_us = 20000
    try:
        interp.interpret(broken.globs)
        code, worker, slot, opcode = mk_mod.read_status("cuda:0")
    finally:
        mk_mod.static_scratch = False
        mk_mod.spin_limit_us = 0
    assert code == 2 and worker == 3 and opcode == 99
    a, b = _both_ways(cfg, workers=16, pos=21, partitions=1)
    assert not mismatches(a, b), mismatches(a, b)


def test_static_scratch_refuses_shapes_beyond_its_size():
    import ctypes

    _, mk_mod = _interpreter()
    lib = mk_mod.load_library()
    args = mk_mod.MkLlamaArgs()
    args.num_layers, args.hidden_size, args.intermediate_size, args.matvec_reduction_size = 512, 4096, 14336, 2048
    assert lib.mk_llama_workspace_bytes(512, 4096, 14336, 2048) > (2 << 20)
    rc = lib.mk_llama_launch_static(ctypes.byref(args), None, None)
    assert rc == -6 and b"static scratch" in lib.mk_llama_last_error()


def test_static_scratch_launch_under_graph_capture():
    """A whole decode step (embedding row of the input token, instruction stream, argmax, barrier
    reset) launched through mk_llama_launch_static inside a captured graph: an allocation would fail
    the capture, the scratch is cleared by a fill kernel (not a memset node), and every replay - with
    eager work and synchronisation in between - gives the bits of the ordinary launch."""
    interp, mk_mod = _interpreter()
    cfg = config_1b_slice(layers=2)
    pos = 70
    model = make_model(cfg, max_len=256)
    fill_kv(model, upto=pos)
    schedule = build_schedule(model, 256, partitions=2)
    schedule.globs.pos_id = pos
    model_plain, plain = mirror_to_gpu(model, schedule)
    model_static, static = mirror_to_gpu(model, schedule)
    token_in = torch.tensor([17], dtype=torch.long, device="cuda:0")
    names = [n for n in plain.globs.mutable_tensor_names() if n != "barriers"]

    out_plain = torch.zeros(1, dtype=torch.long, device="cuda:0")
    interp.interpret_step(plain.globs, model_plain.model.embed_tokens.weight, token_in, out_plain)
    mk_mod.check_status("cuda:0")

    out_static = torch.zeros(1, dtype=torch.long, device="cuda:0")
    embed = model_static.model.embed_tokens.weight
    mk_mod.static_scratch = True
    try:
        # the first call on a device does its one-time set-up (function attributes, the scratch
        # array's address, the look at the instruction tensor): outside the capture
        interp.interpret_step(static.globs, embed, token_in, out_static)
        mk_mod.check_status("cuda:0")
        assert int(out_static) == int(out_plain)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            interp.interpret_step(static.globs, embed, token_in, out_static)
        for replay in range(3):
            # the program's own eager work between the replays: wipe what the step writes
            out_static.zero_()
            static.globs.logits.zero_()
            static.globs.attn_out.zero_()
            static.globs.silu_out.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            mk_mod.check_status("cuda:0")
            assert int(out_static) == int(out_plain), f"replay {replay}"
            report = mismatches(plain.globs, static.globs, names=names, kv_rows=slice(0, pos + 1))
            assert not report, f"replay {replay}: {report}"
            assert int(static.globs.barriers.abs().sum()) == 0
    finally:
        mk_mod.static_scratch = False

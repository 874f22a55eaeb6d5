"""Host-side mirror of the reference's Python surface: model container, rotary
tables, generators, dispatch, and the mk_dir discovery contract."""

import sys
import types

import pytest
import torch

from helpers import build_schedule, config_tiny, fill_kv, make_model
from megakernels_amd import dispatch
from megakernels_amd.generators import MK_Generator, PyTorchGenerator
from megakernels_amd.llama import (
    LlamaConfig, LlamaForCausalLM, interleave_permutation, rope_inverse_frequencies, rope_tables,
)
from megakernels_amd.mk import MK_Interpreter, get_mk_func
from megakernels_amd.model_types import BatchState, ExtraModelConfig
from megakernels_amd.utils import assert_div, get_sm_count, set_sm_count_override


def test_utils():
    assert assert_div(12, 4) == 3
    with pytest.raises(AssertionError):
        assert_div(13, 4)
    set_sm_count_override(132)
    assert get_sm_count("cpu") == 132
    set_sm_count_override(None)
    assert get_sm_count("cpu") == 256  # MI355X default when no GPU is visible
    with pytest.raises(ValueError):
        set_sm_count_override(0)


def test_rope_frequencies_match_transformers_llama3_scaling():
    """The closed-form llama3 scaling against the third-party implementation the reference
    uses (transformers' rope utilities), for both model families."""
    try:
        from transformers import LlamaConfig as HFConfig
        from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS
    except Exception as exc:  # pragma: no cover
        pytest.skip(f"transformers rope utilities not importable: {exc}")
    for cfg in (LlamaConfig.llama_1b(), LlamaConfig.llama_8b()):
        scaling = dict(cfg.rope_scaling)
        hf = HFConfig(hidden_size=cfg.hidden_size, num_attention_heads=cfg.num_attention_heads,
                      num_key_value_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim,
                      rope_theta=cfg.rope_theta, max_position_embeddings=cfg.max_position_embeddings,
                      rope_scaling=scaling)
        try:
            inv_freq, attention_factor = ROPE_INIT_FUNCTIONS["llama3"](hf, "cpu")
        except Exception as exc:  # pragma: no cover - API drift between transformers versions
            pytest.skip(f"transformers llama3 rope init not callable here: {exc}")
        assert attention_factor == 1.0
        ours = rope_inverse_frequencies(cfg)
        assert torch.allclose(ours, inv_freq, rtol=1e-6, atol=0)


def test_rope_tables_layout():
    cfg = config_tiny()
    cos, sin = rope_tables(cfg, 32)
    D = cfg.head_dim
    assert cos.shape == (32, D) and cos.dtype == torch.float32
    assert torch.equal(cos[:, : D // 2], cos[:, D // 2:])            # half-split layout
    assert torch.equal(cos[0], torch.ones(D)) and torch.equal(sin[0], torch.zeros(D))
    perm = interleave_permutation(D)
    assert perm[:4].tolist() == [0, D // 2, 1, D // 2 + 1]
    il = cos[:, perm]
    assert torch.equal(il[:, 0::2], il[:, 1::2])                      # pairs share a frequency
    model = make_model(cfg)
    assert torch.equal(model.model.rope_cos[:32], il)


def test_from_random_is_reproducible_and_tied():
    cfg = config_tiny()
    a, b = make_model(cfg, seed=5), make_model(cfg, seed=5)
    for name in vars(a.stacked_params):
        assert torch.equal(getattr(a.stacked_params, name), getattr(b.stacked_params, name))
    assert a.lm_head.lm_head.weight is a.model.embed_tokens.weight      # tied, as Llama-3.2-1B
    c = make_model(cfg, seed=6)
    assert not torch.equal(a.stacked_params.up_proj, c.stacked_params.up_proj)
    p = a.stacked_params
    L, H, KVH, D = cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    assert p.qkv_proj.shape == (L, (H + 2 * KVH) * D, cfg.hidden_size)
    assert p.down_proj.shape == (L, cfg.hidden_size, cfg.intermediate_size)
    assert a.stacked_kv_cache[0].shape == (L, 1, 256, KVH, D)
    assert abs(float(p.up_proj.float().std()) - 0.02) < 2e-3
    untied = LlamaForCausalLM.from_random(
        LlamaConfig(hidden_size=512, intermediate_size=1024, num_hidden_layers=1, num_attention_heads=8,
                    num_key_value_heads=2, vocab_size=1024, tie_word_embeddings=False, max_position_embeddings=64),
        ExtraModelConfig(interleave_rope=True, max_len_override=16))
    assert untied.lm_head.lm_head.weight is not untied.model.embed_tokens.weight


def test_forward_prefill_equals_token_by_token_decode():
    cfg = config_tiny()
    model = make_model(cfg, max_len=32, seed=1)
    ids = torch.randint(0, cfg.vocab_size, (1, 9), generator=torch.Generator().manual_seed(0))
    full = model(BatchState(input_ids=ids, position_ids=torch.arange(9)))
    kv_full = [c.clone() for c in model.stacked_kv_cache]
    model.setup_caches()
    outs = []
    for t in range(9):
        step = model(BatchState(input_ids=ids[:, t:t + 1], position_ids=torch.tensor([t]), seq_len=t + 1))
        outs.append(step.hidden_states[:, 0])
    stepwise = torch.stack(outs, dim=1)
    assert (stepwise.float() - full.hidden_states.float()).abs().max() <= 2e-2 * full.hidden_states.float().abs().max()
    for a, b in zip(kv_full, model.stacked_kv_cache):
        assert (a[:, :, :9].float() - b[:, :, :9].float()).abs().max() <= 2e-2 * a.float().abs().max()


def test_interleaved_and_half_split_models_agree():
    cfg = config_tiny()
    il = LlamaForCausalLM.from_random(cfg, ExtraModelConfig(interleave_rope=True, max_len_override=16), seed=2)
    hs = LlamaForCausalLM.from_random(cfg, ExtraModelConfig(interleave_rope=False, max_len_override=16), seed=2)
    ids = torch.randint(0, cfg.vocab_size, (1, 6), generator=torch.Generator().manual_seed(3))
    a = il(BatchState(input_ids=ids, position_ids=torch.arange(6)))
    b = hs(BatchState(input_ids=ids, position_ids=torch.arange(6)))
    assert (a.hidden_states.float() - b.hidden_states.float()).abs().max() <= 2e-2 * b.hidden_states.float().abs().max()


class _RecordingInterpreter:
    def __init__(self):
        self.calls = []

    def interpret(self, globs):
        self.calls.append((int(globs.pos_id), globs.barriers.clone(), globs.hidden_states.clone()))
        globs.logits.zero_()
        globs.logits[7] = 1.0
        globs.logits[9] = 1.0  # tie: argmax must pick index 7


def test_mk_generator_loop_semantics():
    """generators.py:121-163: embedding row into hidden_states, barrier fill, pos_id =
    prompt_len + already + i - 1, argmax with first-maximum tie break, token written at src + 1."""
    cfg = config_tiny()
    model = make_model(cfg)
    sched = build_schedule(model, 16)
    interp = _RecordingInterpreter()
    gen = MK_Generator(model, interp, sched, barrier_fill_val=3)
    tokens = torch.zeros(1, 5, dtype=torch.long)
    tokens[0, 0] = 11
    gen.generate(tokens, prompt_len=20, ntok=4, ntok_already_generated=1)
    assert tokens[0].tolist() == [11, 7, 7, 7, 7]
    assert [c[0] for c in interp.calls] == [20, 21, 22, 23]
    assert all(bool((c[1] == 3).all()) for c in interp.calls)
    assert torch.equal(interp.calls[0][2], model.model.embed_tokens.weight[11])
    assert torch.equal(interp.calls[1][2], model.model.embed_tokens.weight[7])
    skipping = MK_Generator(model, interp, sched, skip_mk=True)
    n = len(interp.calls)
    skipping.run(tokens[:, :1], pos_id=3)
    assert len(interp.calls) == n
    gen.replace_with_noops()
    assert int(sched.globs.instructions.abs().sum()) == 0


def test_generate_with_eos_chunks():
    cfg = config_tiny()
    model = make_model(cfg)
    sched = build_schedule(model, 16)
    gen = MK_Generator(model, _RecordingInterpreter(), sched)
    tokens = torch.zeros(1, 40, dtype=torch.long)
    pos, generated = gen.generate_with_eos(tokens, prompt_len=4, ntok=40, eos_token_check_interval=16, eos_token_ids=[7])
    assert (pos, generated) == (1, 16)
    pos, generated = gen.generate_with_eos(tokens, prompt_len=4, ntok=40, eos_token_check_interval=16, eos_token_ids=[99])
    assert (pos, generated) == (40, 39)


def test_pytorch_generator_matches_manual_decode():
    cfg = config_tiny()
    model = make_model(cfg, max_len=32, seed=1)
    ids = torch.randint(0, cfg.vocab_size, (1, 5), generator=torch.Generator().manual_seed(0))
    out = model(BatchState(input_ids=ids, position_ids=torch.arange(5)))
    tokens = torch.zeros(1, 4, dtype=torch.long)
    tokens[0, 0] = out.output_ids[0, -1]
    PyTorchGenerator(model).generate(tokens, prompt_len=5, ntok=3)
    assert tokens.min() >= 0 and tokens.max() < cfg.vocab_size and int(tokens[0, 1:].abs().sum()) > 0


def test_dispatch_and_mk_dir_contract(tmp_path):
    assert type(dispatch.make_schedule_builder("latency")).__name__ == "LatencyScheduleBuilder"
    with pytest.raises(ValueError):
        dispatch.make_schedule_builder("throughput")
    with pytest.raises(NotImplementedError):
        dispatch.make_pyvm_interpreter("latency")
    # mk_dir is put on sys.path and must hold a module `mk_llama` with a callable `mk_llama`
    saved = sys.modules.pop("mk_llama", None)
    saved_path = list(sys.path)
    # the directory is appended (as the reference does), so an earlier entry would win
    sys.path[:] = [p for p in sys.path if not p.rstrip("/").endswith("csrc")]
    try:
        (tmp_path / "mk_llama.py").write_text("def mk_llama(*a, **k):\n    return 'called'\n")
        func = get_mk_func(tmp_path)
        assert func() == "called"
        with pytest.raises(NotImplementedError):
            MK_Interpreter(tmp_path).interpret(None)
    finally:
        sys.modules.pop("mk_llama", None)
        if saved is not None:
            sys.modules["mk_llama"] = saved
        sys.path[:] = saved_path


def test_shim_refuses_cpu_tensors_and_missing_library(monkeypatch):
    sys.modules.pop("mk_llama", None)
    from megakernels_amd.mk import DEFAULT_MK_DIR
    func = get_mk_func(DEFAULT_MK_DIR)
    model = make_model(config_tiny())
    sched = build_schedule(model, 16)
    from megakernels_amd.demos.latency.mk import LatencyMK_Interpreter
    interp = LatencyMK_Interpreter(DEFAULT_MK_DIR)
    with pytest.raises(RuntimeError):
        # no fallback: CPU tensors are refused before anything is launched
        monkeypatch.setattr(torch.cuda, "current_stream", lambda *a, **k: types.SimpleNamespace(cuda_stream=0))
        interp.interpret(sched.globs)
    mod = sys.modules["mk_llama"]
    monkeypatch.setattr(mod, "_lib", None)
    monkeypatch.setattr(mod, "LIBRARY", mod.LIBRARY.with_name("missing.so"))
    with pytest.raises(RuntimeError, match="missing"):
        mod.load_library()


def test_from_pretrained_reads_a_hugging_face_checkpoint_and_matches_its_forward(tmp_path):
    """A checkpoint directory written by the installed third-party `transformers` (random tiny Llama with
    llama3 rope scaling, untied head) is loaded by `from_pretrained`; both the interleaved and the
    half-split model must reproduce the third-party model's logits.  Pins the name mapping, the
    rotary-pair row permutation and the PyTorch forward against an independent implementation."""
    transformers = pytest.importorskip("transformers")
    hf_cfg = transformers.LlamaConfig(
        vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
        num_key_value_heads=2, head_dim=64, max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=500000.0,
        tie_word_embeddings=False, attention_bias=False, mlp_bias=False,
        rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                      "original_max_position_embeddings": 64},
    )
    torch.manual_seed(11)
    hf = transformers.LlamaForCausalLM(hf_cfg).to(torch.float32).eval()
    hf.save_pretrained(tmp_path, safe_serialization=True)
    ids = torch.randint(0, 512, (1, 12), generator=torch.Generator().manual_seed(5))
    with torch.no_grad():
        want = hf(input_ids=ids).logits[0].float()

    for interleave in (True, False):
        ours = LlamaForCausalLM.from_pretrained(
            tmp_path, ExtraModelConfig(interleave_rope=interleave, max_len_override=32), dtype=torch.float32)
        assert ours.config.num_hidden_layers == 2 and ours.lm_head.lm_head.weight is not ours.model.embed_tokens.weight
        out = ours(BatchState(input_ids=ids, position_ids=torch.arange(12)))
        logits = ours.lm_head.lm_head.weight.float() @ _final_norm(ours, out.hidden_states[0].float()).T
        assert (logits.T - want).abs().max() <= 2e-4 * want.abs().max(), interleave
        assert out.output_ids[0].tolist() == want.argmax(-1).tolist()


def _final_norm(model, hidden):
    w = model.lm_head.input_norm.weight.float()
    return w * hidden * torch.rsqrt(hidden.pow(2).mean(-1, keepdim=True) + model.config.rms_norm_eps)


def _tiny_chat_checkpoint(tmp_path):
    """A checkpoint directory as a user would have it: weights and config written by the installed
    third-party `transformers`, a word-level tokenizer with a chat template, a generation config."""
    transformers = pytest.importorskip("transformers")
    tokenizers = pytest.importorskip("tokenizers")
    words = ["<pad>", "<bos>", "<eos>", "<user>", "<assistant>", "hi", "tell", "me", "a", "joke", "about", "cookies",
             "why", "did", "the", "cookie", "cry"]
    vocab = {w: i for i, w in enumerate(words)}
    tok = tokenizers.Tokenizer(tokenizers.models.WordLevel(vocab, unk_token="<pad>"))
    tok.pre_tokenizer = tokenizers.pre_tokenizers.WhitespaceSplit()
    fast = transformers.PreTrainedTokenizerFast(tokenizer_object=tok, bos_token="<bos>", eos_token="<eos>", pad_token="<pad>")
    fast.chat_template = ("<bos>{% for m in messages %} <{{ m['role'] }}> {{ m['content'] }} <eos>{% endfor %}"
                          "{% if add_generation_prompt %} <assistant>{% endif %}")
    fast.save_pretrained(tmp_path)
    hf_cfg = transformers.LlamaConfig(
        vocab_size=64, hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=2,
        num_key_value_heads=1, head_dim=64, max_position_embeddings=128, rms_norm_eps=1e-5, rope_theta=500000.0,
        tie_word_embeddings=True, attention_bias=False, mlp_bias=False, eos_token_id=2, bos_token_id=1)
    torch.manual_seed(3)
    transformers.LlamaForCausalLM(hf_cfg).eval().save_pretrained(tmp_path, safe_serialization=True)
    (tmp_path / "generation_config.json").write_text('{"eos_token_id": [2, 0]}')
    return vocab


def test_prompt_encoding_and_eos_ids_of_a_local_checkpoint(tmp_path):
    from megakernels_amd.scripts.text import encode_messages, encode_prompt, eos_token_ids, load_tokenizer

    vocab = _tiny_chat_checkpoint(tmp_path)
    assert load_tokenizer(tmp_path / "nowhere") is None
    tok = load_tokenizer(tmp_path)
    plain = encode_prompt(tok, "tell me a joke", chat=False)
    assert plain.tolist() == [[vocab[w] for w in "tell me a joke".split()]]
    chat = encode_prompt(tok, "tell me a joke", chat=True)
    want = "<bos> <user> tell me a joke <eos> <assistant>".split()
    assert chat.tolist() == [[vocab[w] for w in want]]
    two = encode_messages(tok, [{"role": "user", "content": "hi"}, {"role": "assistant", "content": "why"},
                                {"role": "user", "content": "joke"}])
    assert two.shape[1] == 1 + 3 * 2 + 3 + 1
    assert eos_token_ids(tmp_path, tok) == [2, 0]
    (tmp_path / "generation_config.json").unlink()
    assert eos_token_ids(tmp_path, tok) == [2]          # from config.json


def test_repl_conversation_on_the_pytorch_generator(tmp_path):
    """The chat loop's core with the plain PyTorch generator on the CPU: each turn re-renders the whole
    conversation, stops at an end-of-sequence id, and a second turn sees the first one's answer."""
    from megakernels_amd.generators import PyTorchGenerator
    from megakernels_amd.scripts.llama_repl import Conversation, parse_args
    from megakernels_amd.scripts.text import eos_token_ids, load_tokenizer

    _tiny_chat_checkpoint(tmp_path)
    tok = load_tokenizer(tmp_path)
    model = LlamaForCausalLM.from_pretrained(tmp_path, ExtraModelConfig(interleave_rope=True, max_len_override=96))
    chat = Conversation(model, PyTorchGenerator(model), tok, eos_token_ids(tmp_path, tok), max_tokens_per_turn=24)
    text, generated, seconds = chat.say("tell me a joke about cookies")
    assert isinstance(text, str) and 1 <= generated <= 23 and seconds > 0
    ids = chat.output_tokens[0].tolist()
    stops = [i for i, t in enumerate(ids[: generated + 1]) if t in (0, 2)]
    # the reply ends at the first end-of-sequence id, if one was produced within the chunks that ran
    assert text == tok.decode(ids[: stops[0] if stops else 24], skip_special_tokens=True)
    first_len = len(chat.messages)
    chat.say("why")
    assert first_len == 2 and len(chat.messages) == 4 and chat.messages[1]["role"] == "assistant"
    with pytest.raises(RuntimeError, match="does not fit the KV cache"):
        Conversation(model, PyTorchGenerator(model), tok, [2], max_tokens_per_turn=200).say("hi")
    cfg = parse_args([f"model={tmp_path}", "mode=torch", "max_tokens_per_turn=8", "print_prompt_len=true"])
    assert cfg.mode == "torch" and cfg.max_tokens_per_turn == 8 and cfg.print_prompt_len is True
    with pytest.raises(SystemExit):
        parse_args(["mode=mk"])


def test_timing_records_in_the_reference_event_slots():
    """scripts/timeline.reference_event_layout: the kernel stamps the reference's event slots
    (include/util.cuh:215-246) itself, with the low 32 bits of one device clock; the re-laid record holds
    the same events as ticks since the first instruction started - also across a wrap of the 32-bit
    clock - with the stages only the reference has (slots 1-3) set to the start, unstamped slots zero."""
    from megakernels_amd.scripts import timeline as tl

    ins = torch.zeros(2, 3, 32, dtype=torch.int32)
    ins[0, 0, 0], ins[0, 1, 0], ins[1, 0, 0] = 1, 6, 2          # worker 1 has two NoOps
    raw = torch.zeros(2, 3, 128, dtype=torch.int64)
    base = (1 << 32) - 50                                         # the clock wraps during the launch

    def record(w, s, opcode, **at):
        raw[w, s, tl.OPCODE] = opcode
        for name, tick in at.items():
            raw[w, s, getattr(tl, name)] = base + tick

    record(0, 0, 1, START=0, DEP_READY=10, DONE_GMEM_WAIT=10, INPUT_READY=20, LAUNCHER_START=20, COMPUTE_DONE=70,
           AT_GMEM_STORE=75, DONE_GMEM_STORE=85, OUTPUT_READY=88, END=90, FIRST_LOAD=2, FIRST_USE=21, LAST_USE=66)
    raw[0, 0, tl.CONSUMER_START + 2 * 3] = base + 22               # consumer wave 3: first row ...
    raw[0, 0, tl.CONSUMER_START + 2 * 3 + 1] = base + 69           # ... and last row done
    record(0, 1, 6, START=100, DEP_READY=100, INPUT_READY=130, COMPUTE_DONE=400, DONE_GMEM_STORE=415, END=420)
    record(1, 0, 2, START=5, DEP_READY=40, INPUT_READY=45, COMPUTE_DONE=300, OUTPUT_READY=309, END=310)
    timings = (raw & 0xFFFFFFFF).to(torch.int32)                 # what the kernel stores
    out = tl.reference_event_layout(timings, ins)
    assert out.shape == timings.shape and out.dtype == torch.int32
    assert out[0, 0, 0] == 0 and out[0, 0, 4] == 90 and out[0, 0, 45] == 10 and out[0, 0, 7] == 20 and out[0, 0, 46] == 75
    assert out[0, 0, 47] == 85 and out[0, 0, 54] == 88 and out[0, 0, 48] == 2 and out[0, 0, 49] == 21 and out[0, 0, 52] == 66
    assert out[0, 0, 11 + 6] == 22 and out[0, 0, 11 + 7] == 69 and out[0, 0, 11] == 0     # wave 0 had no row
    assert out[0, 1, 0] == 100 and out[0, 1, 47] == 415 and out[0, 1, 46] == 0 and out[1, 0, 0] == 5 and out[1, 0, 54] == 309
    # the reference's fetch / page / semaphore stages: over when the instruction starts
    assert [int(out[0, 1, k]) for k in (1, 2, 3)] == [100, 100, 100] and int(out[1, 0, 2]) == 5
    assert int(out[0, 0, tl.OPCODE]) == 1 and int(out[1, 0, tl.OPCODE]) == 2
    assert int(out[1, 1:].abs().sum()) == 0 and int(out[0, 2].abs().sum()) == 0
    unused = [i for i in range(128) if i not in tl.TIME_SLOTS and i not in tl.REFERENCE_ONLY_STAGES and i != tl.OPCODE]
    assert int(out[:, :, unused].abs().sum()) == 0
    t, stamped = tl.microseconds(timings.numpy())
    assert abs(t[0, 1, tl.END] - 4.2) < 1e-9 and bool(stamped[0, 0, tl.FIRST_USE]) and not bool(stamped[0, 1, tl.FIRST_USE])

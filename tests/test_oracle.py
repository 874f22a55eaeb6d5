"""Pins for the CPU checker (oracle/mk_oracle.c).

The reference ships no golden vectors for this path, so every solver of the
checker is pinned against what the mathematics fixes: fp64 brute force on small
inputs (a dropped term, a wrong sign, a transposed operand or a shifted index
fails these), special cases that reduce to library routines (softmax attention
= torch SDPA, RMSNorm, SiLU), invariants (split-KV partitions + reduction = one
partition; rotation preserves the norm; position 0 is the identity), the closed
form of the barrier tensor after a full step, a plain Llama decode step, and a
second restatement written with the torch operations the reference uses
(oracle/pyvm_torch.py).  Tolerances are stated where they apply; they are bf16
rounding (2^-8 relative) unless noted."""

import math

import numpy as np
import pytest
import torch

from helpers import build_schedule, config_1b_slice, config_8b_slice, config_tiny, fill_kv, make_model
from megakernels_amd.demos.latency.instructions import (
    AttentionReduction, DownProjResidual, LayerNorm_QKV_MatVecRopeAppend, LayerNormDoubleMatVecSiLU,
    O_ProjResidual, PartialAttention, RMS_LM_Head,
)
from megakernels_amd.model_types import BatchState
from oracle import pyvm, pyvm_torch

BF16_EPS = 2.0 ** -8


def f64(t):
    return t.detach().to(torch.float64).numpy()


def bf16_round(x: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).to(torch.bfloat16).to(torch.float64).numpy()


def ulp_diff_f32(a, b):
    ai = np.asarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    bi = np.asarray(b, dtype=np.float32).view(np.int32).astype(np.int64)
    return np.abs(ai - bi)


def fresh(cfg, workers=16, pos=37, partitions=1, seed=0, hidden_scale=1.0, **kw):
    model = make_model(cfg, max_len=max(256, pos + 8), seed=seed)
    fill_kv(model, upto=pos)
    sched = build_schedule(model, workers, partitions=partitions, **kw)
    g = sched.globs
    gen = torch.Generator().manual_seed(11)
    g.hidden_states.copy_((torch.randn(cfg.hidden_size, generator=gen) * hidden_scale).to(torch.bfloat16))
    g.pos_id = pos
    return model, sched, g


def rms_ref(x, w, eps):
    x = f64(x)
    normed = bf16_round(x / np.sqrt((x * x).mean() + eps))
    return bf16_round(f64(w) * normed)


# ---------------------------------------------------------------------------------------------
# scalar kernels
# ---------------------------------------------------------------------------------------------


def test_bf16_rounding_matches_torch():
    lib = pyvm.load_lib()
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    edge = np.array([0x00000000, 0x80000000, 0x3F800000, 0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001,
                     0x7F7FFFFF, 0x7F800000, 0xFF800000, 0x00000001, 0x00008000, 0x0000FFFF, 0x7F7F8000], dtype=np.uint32)
    vals = np.concatenate([bits, edge]).view(np.float32)
    vals = vals[~np.isnan(vals)]
    want = torch.from_numpy(vals.copy()).to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16)
    got = np.array([lib.mk_oracle_f32_to_bf16(float(v)) for v in vals[:20000]], dtype=np.uint16)
    assert np.array_equal(got, want[:20000])
    got_edge = np.array([lib.mk_oracle_f32_to_bf16(float(v)) for v in vals[-len(edge):]], dtype=np.uint16)
    assert np.array_equal(got_edge, want[-len(edge):])


def test_exp_exp2_log2_accuracy():
    """<= 2 ulp against float64 libm on the ranges the VM uses (softmax arguments <= 0, silu
    arguments of any sign, partition sums >= 1)."""
    lib = pyvm.load_lib()
    xs = np.concatenate([np.linspace(-80, 0, 4001), np.linspace(0, 60, 1501), [-86.0, -1e-7, 1e-7, 0.0]]).astype(np.float32)
    got = np.array([lib.mk_oracle_expf(float(x)) for x in xs], dtype=np.float32)
    want = np.exp(xs.astype(np.float64)).astype(np.float32)
    assert ulp_diff_f32(got, want).max() <= 2
    assert lib.mk_oracle_expf(-100.0) == 0.0 and lib.mk_oracle_expf(0.0) == 1.0
    xs = np.concatenate([np.linspace(-120, 0, 3001), np.linspace(0, 20, 501)]).astype(np.float32)
    got = np.array([lib.mk_oracle_exp2f(float(x)) for x in xs], dtype=np.float32)
    assert ulp_diff_f32(got, np.exp2(xs.astype(np.float64)).astype(np.float32)).max() <= 2
    assert lib.mk_oracle_exp2f(float("-inf")) == 0.0 and lib.mk_oracle_exp2f(-3.0) == 0.125
    xs = np.concatenate([np.linspace(1, 70000, 5001), np.linspace(0.01, 1, 500)]).astype(np.float32)
    got = np.array([lib.mk_oracle_log2f(float(x)) for x in xs], dtype=np.float64)
    want = np.log2(xs.astype(np.float64))
    assert np.abs(got - want).max() <= 2e-6
    assert lib.mk_oracle_log2f(8.0) == 3.0 and lib.mk_oracle_log2f(1.0) == 0.0


def _bf16_parts(h):
    """(sign, exponent, significand) of a finite bf16 bit pattern: value = (-1)^s * m * 2^(e - 127 - 7)"""
    s, e, m = (h >> 15) & 1, (h >> 7) & 0xFF, h & 0x7F
    return (s, 1, m) if e == 0 else (s, e, m | 0x80)


def dot2_by_the_words(a, b, acc_bits):
    """acc + a.lo*b.lo + a.hi*b.hi for finite operands, following the words of the definition with exact
    rationals (no shifts, no two's complement): truncation is floor(), rounding is Python's exact
    float(Fraction) followed by a float32 cast that is checked to be exact or a single rounding."""
    from fractions import Fraction
    from math import floor

    prods = []
    for lo in (True, False):
        x, y = (a & 0xFFFF, b & 0xFFFF) if lo else (a >> 16, b >> 16)
        (sx, ex, mx), (sy, ey, my) = _bf16_parts(x), _bf16_parts(y)
        if mx * my:
            prods.append((-1 if sx ^ sy else 1, mx * my, ex + ey - 127))
    sc, ec, mc = acc_bits >> 31, (acc_bits >> 23) & 0xFF, acc_bits & 0x7FFFFF
    ec, mc = (1, mc) if ec == 0 else (ec, mc | 0x800000)
    c = Fraction(-mc if sc else mc) * Fraction(2) ** (ec - 127 - 23)
    L = max(ec - 32, -30)
    P = Fraction(0)
    if prods:
        emax = max(e for _, _, e in prods)
        unit = Fraction(2) ** (emax - 24 - 127)
        for sign, m, e in prods:
            mag = Fraction(m) * Fraction(2) ** (e - 127 - 14)
            P += sign * floor(mag / unit) * unit  # cut off towards zero below 2^(emax - 24)
        L = max(L, emax - 24)
    unit = Fraction(2) ** (L - 127)
    t = floor(P / unit) + floor(c / unit)  # towards minus infinity
    while abs(t) >= 1 << 32:
        t = floor(Fraction(t, 2))
        unit *= 2
    if t == 0:
        return np.float32(0.0)
    # one rounding to nearest even: |t| < 2^32 fits a double exactly, so does t * 2^(L - 127)
    r = np.float32(float(t * unit))
    return np.float32(0.0) if r == 0 else r  # also when the rounding went to zero


def test_dot2_definition_against_the_instructions_results():
    """tests/golden/dot2_vectors.npz holds results of the GPU instruction (written by
    tests/golden/make_dot2_vectors.py on an MI355X); the C definition must reproduce every one of them,
    and so must the restatement in exact rationals on the finite cases."""
    from pathlib import Path

    import dot2_cases

    v = np.load(Path(__file__).parent / "golden" / "dot2_vectors.npz")
    a, b, acc, out = v["a"], v["b"], v["acc"], v["out"]
    assert len(a) >= 50000
    got = pyvm.dot2(a, b, acc.view(np.float32)).view(np.uint32)
    bad = np.flatnonzero(~dot2_cases.same_results(got, out))
    assert bad.size == 0, [(hex(a[i]), hex(b[i]), hex(acc[i]), hex(out[i]), hex(got[i])) for i in bad[:5]]
    # the clause-by-clause form alone, and both forms on fresh operands of every class
    assert dot2_cases.same_results(pyvm.dot2(a, b, acc.view(np.float32), general=True).view(np.uint32), out).all()
    rng = np.random.default_rng(99)
    for gen in dot2_cases.CLASSES:
        x, y, z = (np.ascontiguousarray(t, dtype=np.uint32) for t in gen(rng, 200000))
        short = pyvm.dot2(x, y, z.view(np.float32)).view(np.uint32)
        full = pyvm.dot2(x, y, z.view(np.float32), general=True).view(np.uint32)
        assert dot2_cases.same_results(short, full).all(), gen.__name__
    # every class is present and none is trivial: results differ from a fused multiply-add chain somewhere
    per = int(v["per_class"])
    assert len(a) == per * len(v["classes"]) and list(v["classes"]) == [g.__name__ for g in dot2_cases.CLASSES]

    def finite_bf(h):
        return ((h >> 7) & 0xFF) != 0xFF

    checked = 0
    for i in range(0, len(a), 7):
        ai, bi, ci = int(a[i]), int(b[i]), int(acc[i])
        if not (finite_bf(ai & 0xFFFF) and finite_bf(ai >> 16) and finite_bf(bi & 0xFFFF) and finite_bf(bi >> 16)) or ((ci >> 23) & 0xFF) == 0xFF:
            continue
        if not np.isfinite(np.array([out[i]], dtype=np.uint32).view(np.float32)[0]):
            continue  # a product beyond the fp32 range: the IEEE clause
        want = dot2_by_the_words(ai, bi, ci)
        assert np.array([want]).view(np.uint32)[0] == out[i], (hex(ai), hex(bi), hex(ci), hex(out[i]), want)
        checked += 1
    assert checked > 5000


def test_dot2_special_values():
    inf, nan = 0x7F80, 0x7FC0
    one, two, mone = 0x3F80, 0x4000, 0xBF80
    f = lambda a, b, c: pyvm.dot2(np.array([a], np.uint32), np.array([b], np.uint32), np.array([c], np.float32))[0]
    assert f(one | (one << 16), two | (two << 16), 0.5) == 4.5
    assert f(one | (mone << 16), one | (one << 16), -0.0) == 0.0 and not np.signbit(f(one | (mone << 16), one | (one << 16), -0.0))
    assert np.isinf(f(inf | (one << 16), one | (one << 16), 1.0))
    assert np.isnan(f(inf | (one << 16), one | (mone << 16) | 0, np.float32(-np.inf)))
    assert np.isnan(f(nan, one, 0.0))
    huge = 0x7F00  # 1.7e38
    assert np.isinf(f(huge | (one << 16), huge | (one << 16), 0.0))           # product beyond fp32: infinity
    assert np.isnan(f(huge | (huge << 16), huge | ((huge | 0x8000) << 16), 0.0))  # +inf + -inf


def test_dot_column_order():
    lib = pyvm.load_lib()
    rng = np.random.default_rng(1)
    import ctypes
    for K in (512, 2048, 4096):
        w = torch.from_numpy(rng.standard_normal(K).astype(np.float32)).to(torch.bfloat16)
        x = torch.from_numpy(rng.standard_normal(K).astype(np.float32)).to(torch.bfloat16).float().contiguous()
        got = lib.mk_oracle_dot(ctypes.cast(w.data_ptr(), pyvm._U16P), ctypes.cast(x.data_ptr(), pyvm._F32P), K)
        want = float(f64(w) @ f64(x))
        assert abs(got - want) <= 1e-5 * math.sqrt(K) * 4
        # the documented order: accumulator c takes the element pairs j*256 + c in order of j through the
        # two-element dot product, then a pairwise tree over the 256 accumulators
        wb = w.view(torch.int16).numpy().astype(np.uint16).astype(np.uint32)
        xb = (x.numpy().view(np.uint32) >> 16).astype(np.uint32)
        acc = np.zeros(256, dtype=np.float32)
        for j in range(0, K, 512):
            pairs = j + 2 * np.arange(256)
            acc = pyvm.dot2(wb[pairs] | (wb[pairs + 1] << 16), xb[pairs] | (xb[pairs + 1] << 16), acc)
        s = 1
        while s < 256:
            for i in range(0, 256, 2 * s):
                acc[i] = np.float32(acc[i] + acc[i + s])
            s *= 2
        assert np.float32(got) == acc[0]
    # exact case: small integers sum exactly in any order
    w = torch.arange(512, dtype=torch.float32).remainder(7).sub(3).to(torch.bfloat16)
    x = torch.arange(512, dtype=torch.float32).remainder(5).sub(2).contiguous()
    got = lib.mk_oracle_dot(ctypes.cast(w.data_ptr(), pyvm._U16P), ctypes.cast(x.data_ptr(), pyvm._F32P), 512)
    assert got == float((w.float() * x).sum())


# ---------------------------------------------------------------------------------------------
# solvers against fp64 brute force
# ---------------------------------------------------------------------------------------------


def test_qkv_rope_append_bruteforce():
    cfg = config_tiny()
    model, sched, g = fresh(cfg, pos=37)
    H, KVH, D, hid = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.hidden_size
    layer = 0
    x = rms_ref(g.hidden_states, g.attn_ln_weights[layer], g.rms_norm_eps)
    y = bf16_round(f64(g.qkv_proj_weights[layer]) @ x)  # matvec -> bf16
    cos, sin = f64(g.rope_cos[37]), f64(g.rope_sin[37])
    want = y.copy()
    for head in range(H + KVH):  # q and k heads rotate adjacent pairs; v untouched
        seg = y[head * D:(head + 1) * D]
        rot = np.empty_like(seg)
        rot[0::2] = seg[0::2] * cos[0::2] - seg[1::2] * sin[0::2]
        rot[1::2] = seg[1::2] * cos[1::2] + seg[0::2] * sin[1::2]
        want[head * D:(head + 1) * D] = rot
    want = bf16_round(want)
    k_before = g.k_cache.clone()
    ins = [i for i in sched.get_linear_instructions() if i.opcode() == 1 and i.layer_idx == 0]
    pyvm.interpret(g, ins)
    got = np.concatenate([f64(g.post_ln_rope_q), f64(g.k_cache[0, 0, 37]).reshape(-1), f64(g.v_cache[0, 0, 37]).reshape(-1)])
    # one bf16 ulp where the fp32 accumulation order moves a value across a rounding boundary
    tol = BF16_EPS * np.maximum(np.abs(want), 1e-3) * 1.01
    assert (np.abs(got - want) <= tol).all()
    assert (np.abs(got - want) > 0).mean() < 0.02
    # only row pos_id of layer 0 changed
    g.k_cache[0, 0, 37] = k_before[0, 0, 37]
    assert torch.equal(g.k_cache, k_before)
    assert g.barriers[0, 0].tolist() == [D // 16] * (H + 2 * KVH)


def test_rope_invariants():
    """Rotation preserves each pair's norm; position 0 is the identity; the interleaved layout on
    permuted weights equals the half-split (Hugging Face) layout on the original weights."""
    from megakernels_amd.llama import (
        apply_rotary_pos_emb, apply_rotary_pos_emb_interleaved, interleave_permutation, rope_tables,
    )
    cfg = config_tiny()
    cos, sin = rope_tables(cfg, 64)
    perm = interleave_permutation(cfg.head_dim)
    q = torch.randn(1, 5, 3, cfg.head_dim, dtype=torch.float64)
    pos = torch.tensor([0, 1, 7, 33, 63])
    c, s = cos[pos].double(), sin[pos].double()
    ref_q, _ = apply_rotary_pos_emb(q, q, c, s, unsqueeze_dim=-2)
    il_q, _ = apply_rotary_pos_emb_interleaved(q[..., perm], q[..., perm], c[:, perm], s[:, perm], unsqueeze_dim=-2)
    assert torch.allclose(il_q, ref_q[..., perm], atol=1e-12)
    assert torch.allclose(il_q[:, 0], q[:, 0][..., perm], atol=0)  # position 0
    pairs = il_q.reshape(1, 5, 3, -1, 2).norm(dim=-1)
    assert torch.allclose(pairs, q[..., perm].reshape(1, 5, 3, -1, 2).norm(dim=-1), atol=1e-9)


def _attention_ref(g, layer, kvh, t0, t1):
    G = g.num_attention_heads // g.num_kv_heads
    q = f64(g.post_ln_rope_q).reshape(g.num_attention_heads, -1)[kvh * G:(kvh + 1) * G]
    k = f64(g.k_cache[layer, 0, t0:t1, kvh])
    v = f64(g.v_cache[layer, 0, t0:t1, kvh])
    s = (q @ k.T) * g.attn_scale
    m = s.max(axis=-1, keepdims=True)
    p = np.exp(s - m)
    l = p.sum(axis=-1, keepdims=True)
    return (p / l) @ v, (np.log2(l) + m * math.log2(math.e)).reshape(-1)


@pytest.mark.parametrize("cfg_fn", [config_tiny, lambda: config_8b_slice(layers=1, vocab=1024, inter=2048)])
def test_partial_attention_bruteforce(cfg_fn):
    cfg = cfg_fn()
    workers = 16 if cfg.hidden_size == 512 else 64
    model, sched, g = fresh(cfg, workers=workers, pos=150)
    gen = torch.Generator().manual_seed(5)
    g.post_ln_rope_q.copy_(torch.randn(g.post_ln_rope_q.shape, generator=gen).to(torch.bfloat16))
    KVH, H = cfg.num_key_value_heads, cfg.num_attention_heads
    g.barriers[0, 0] = cfg.head_dim // 16
    for kvh in (0, KVH - 1):
        pyvm.interpret(g, [PartialAttention(0, kvh, 1, 0)])
        want, _ = _attention_ref(g, 0, kvh, 0, 151)
        G = H // KVH
        got = f64(g.attn_out).reshape(H, -1)[kvh * G:(kvh + 1) * G]
        assert np.abs(got - bf16_round(want)).max() <= BF16_EPS * np.abs(want).max() * 1.01
    assert int(g.barriers[0, 2, 0]) == 2 * (H // KVH)
    # the same thing through torch's SDPA
    q = g.post_ln_rope_q.view(1, H, 1, -1).float()
    k = g.k_cache[0, :, :151].transpose(1, 2).float()
    v = g.v_cache[0, :, :151].transpose(1, 2).float()
    sdpa = torch.nn.functional.scaled_dot_product_attention(q, k, v, enable_gqa=True).reshape(H, -1)
    got_all = g.attn_out.view(H, -1).float()
    G = H // KVH
    for kvh in (0, KVH - 1):
        sl = slice(kvh * G, (kvh + 1) * G)
        assert (got_all[sl] - sdpa[sl]).abs().max() <= BF16_EPS * sdpa[sl].abs().max() * 1.5


def test_split_kv_equals_single_partition():
    """Partitions + log-sum-exp reduction reproduce the unsplit softmax (fp32 rounding only); an
    empty partition yields zeros and lse = -inf and drops out of the merge."""
    cfg = config_tiny()
    model, sched, g = fresh(cfg, pos=100, partitions=1)
    gen = torch.Generator().manual_seed(6)
    g.post_ln_rope_q.copy_(torch.randn(g.post_ln_rope_q.shape, generator=gen).to(torch.bfloat16))
    want, want_lse = _attention_ref(g, 1, 1, 0, 101)
    for P in (2, 3, 7, 9):  # 7 blocks: P = 9 leaves two partitions empty
        model2, sched2, g2 = fresh(cfg, pos=100, partitions=P)
        g2.post_ln_rope_q.copy_(g.post_ln_rope_q)
        g2.barriers[1, 0] = 4
        pyvm.interpret(g2, [PartialAttention(1, 1, P, p) for p in range(P)])
        lses = f64(g2.attn_lse_intermediates[4:8, :P])
        outs = f64(g2.attn_out_intermediates[4:8, :P])
        if P == 9:
            assert np.isneginf(lses[:, 7:]).all() and (outs[:, 7:] == 0).all()
        # each partition's lse is the base-2 log-sum-exp of its slice
        _, lse0 = _attention_ref(g2, 1, 1, 0, min(101, math.ceil(math.ceil(101 / 16) / P) * 16))
        lse_tol = 4 * 2.0 ** -23 * np.abs(want_lse).max() + 1e-6  # fp32 rounding at the value's magnitude
        assert np.abs(lses[:, 0] - lse0).max() <= lse_tol
        g2.barriers[1, 1, 4] = P
        pyvm.interpret(g2, [AttentionReduction(1, 4, P, True, list(range(P)), None)])
        got = f64(g2.attn_out).reshape(cfg.num_attention_heads, -1)[4:8]
        assert np.abs(got - bf16_round(want)).max() <= BF16_EPS * np.abs(want).max() * 1.01
        assert int(g2.barriers[1, 2, 0]) == 4
        # merged lse of all partitions = lse of the whole range
        merged = np.log2(np.exp2(lses - lses.max(axis=1, keepdims=True)).sum(axis=1)) + lses.max(axis=1)
        assert np.abs(merged - want_lse).max() <= lse_tol


@pytest.mark.parametrize("P", [32, 64])
def test_reduction_tree_equals_single_partition(P):
    """A whole layer's attention through a two-level reduction tree (P partitions, first-level merges,
    terminal merge) reproduces the unsplit softmax, and leaves the counters in their closed form:
    row 1 holds the partitions plus the first-level merges of each head, row 2 the heads."""
    from megakernels_amd.demos.latency.scheduler import reduction_tree_runs

    cfg = config_tiny()
    pos = 16 * P + 5                      # every partition has tokens, the last one five

    def fresh(*args, **kw):
        # the newest position is normally written by the QKV instruction, which this test leaves out
        model, sched, g = globals()["fresh"](*args, **kw)
        row = torch.Generator().manual_seed(9)
        for cache in model.stacked_kv_cache:
            cache[:, :, pos] = torch.randn(cache[:, :, pos].shape, generator=row).to(cache.dtype)
        return model, sched, g

    model, sched, g = fresh(cfg, workers=96, pos=pos, partitions=1)
    gen = torch.Generator().manual_seed(6)
    g.post_ln_rope_q.copy_(torch.randn(g.post_ln_rope_q.shape, generator=gen).to(torch.bfloat16))
    want = [_attention_ref(g, 1, kv, 0, pos + 1)[0] for kv in range(cfg.num_key_value_heads)]
    model2, sched2, g2 = fresh(cfg, workers=96, pos=pos, partitions=P)
    g2.post_ln_rope_q.copy_(g.post_ln_rope_q)
    g2.barriers[1, 0] = 4
    chain = [i for i in sched2.get_linear_instructions() if i.opcode() in (2, 3) and i.layer_idx == 1]
    pyvm.interpret(g2, chain)
    got = f64(g2.attn_out).reshape(cfg.num_attention_heads, -1)
    for kv in range(cfg.num_key_value_heads):
        ref = want[kv]
        assert np.abs(got[4 * kv : 4 * kv + 4] - bf16_round(ref)).max() <= BF16_EPS * np.abs(ref).max() * 1.01
    runs = reduction_tree_runs(P)
    assert len(runs) > 1
    assert (g2.barriers[1, 1, : cfg.num_attention_heads] == P + len(runs)).all()
    assert int(g2.barriers[1, 2, 0]) == cfg.num_attention_heads
    # the torch restatement agrees on the counters and, within rounding, on the result
    model3, sched3, g3 = fresh(cfg, workers=96, pos=pos, partitions=P)
    g3.post_ln_rope_q.copy_(g.post_ln_rope_q)
    g3.barriers[1, 0] = 4
    pyvm_torch.interpret(g3, [i for i in sched3.get_linear_instructions() if i.opcode() in (2, 3) and i.layer_idx == 1])
    assert torch.equal(g3.barriers, g2.barriers)
    assert np.abs(f64(g3.attn_out) - f64(g2.attn_out)).max() <= 2e-2 * np.abs(f64(g2.attn_out)).max()


def test_attention_reduction_nonterminal_and_list_order():
    cfg = config_tiny()
    model, sched, g = fresh(cfg, pos=100, partitions=4)
    gen = torch.Generator().manual_seed(7)
    H, D = cfg.num_attention_heads, cfg.head_dim
    g.attn_lse_intermediates[:, :4] = torch.randn(H, 4, generator=gen) * 3
    g.attn_out_intermediates[:, :4] = torch.randn(H, 4, D, generator=gen)
    g.barriers[0, 1, 0] = 4
    lses, outs = f64(g.attn_lse_intermediates[0:4, :4]), f64(g.attn_out_intermediates[0:4, :4])
    pyvm.interpret(g, [AttentionReduction(0, 0, 4, False, [2, 0], 5)])
    w = np.exp2(lses[:, [2, 0]] - lses[:, [2, 0]].max(axis=1, keepdims=True))
    want = (outs[:, [2, 0]] * w[..., None]).sum(axis=1) / w.sum(axis=1, keepdims=True)
    assert np.abs(f64(g.attn_out_intermediates[0:4, 5]) - want).max() <= 1e-6
    want_lse = lses[:, [2, 0]].max(axis=1) + np.log2(w.sum(axis=1))
    assert np.abs(f64(g.attn_lse_intermediates[0:4, 5]) - want_lse).max() <= 1e-6


def test_matvec_residual_and_order_of_partial_sums():
    cfg = config_8b_slice(layers=1, vocab=1024, inter=6144)  # 2 O groups, 3 down groups
    model, sched, g = fresh(cfg, workers=64, pos=10)
    gen = torch.Generator().manual_seed(8)
    g.attn_out.copy_(torch.randn(cfg.hidden_size, generator=gen).to(torch.bfloat16))
    g.silu_out.copy_(torch.randn(cfg.intermediate_size, generator=gen).to(torch.bfloat16))
    h0 = f64(g.hidden_states).copy()
    g.barriers[0, 2, 0] = cfg.num_attention_heads
    rows = slice(32, 64)
    pyvm.interpret(g, [O_ProjResidual(0, 2, 4, 0), O_ProjResidual(0, 2, 4, 1)])
    W = f64(g.o_proj_weights[0])
    want = h0[rows]
    for grp in range(2):
        cols = slice(grp * 2048, (grp + 1) * 2048)
        part = bf16_round(W[rows, cols] @ f64(g.attn_out)[cols])
        want = bf16_round(want + part)
    got = f64(g.hidden_states)[rows]
    assert np.abs(got - want).max() <= BF16_EPS * np.abs(want).max() * 1.01
    assert (got != want).mean() < 0.1
    assert np.array_equal(f64(g.hidden_states)[:32], h0[:32])
    assert int(g.barriers[0, 3, 0]) == 4
    # down projection, groups applied 0, 1, 2: bf16(bf16(bf16(h + p0) + p1) + p2)
    h1 = f64(g.hidden_states).copy()
    g.barriers[0, 4, 0] = cfg.intermediate_size // 16
    pyvm.interpret(g, [DownProjResidual(0, 0, 1, grp) for grp in range(3)])
    Wd = f64(g.down_proj_weights[0])
    want = h1[:16]
    for grp in range(3):
        cols = slice(grp * 2048, (grp + 1) * 2048)
        want = bf16_round(want + bf16_round(Wd[:16, cols] @ f64(g.silu_out)[cols]))
    assert np.abs(f64(g.hidden_states)[:16] - want).max() <= BF16_EPS * np.abs(want).max() * 1.01
    assert int(g.barriers[0, 5, 0]) == 3


def test_upgate_silu_and_lm_head_bruteforce():
    cfg = config_tiny()
    model, sched, g = fresh(cfg, pos=5)
    g.barriers[1, 3, 0] = g.o_proj_total_jobs()
    pyvm.interpret(g, [LayerNormDoubleMatVecSiLU(1, [0, 3, 63])])
    x = rms_ref(g.hidden_states, g.mlp_ln_weights[1], g.rms_norm_eps)
    for b in (0, 3, 63):
        rows = slice(b * 16, b * 16 + 16)
        up = bf16_round(f64(g.up_proj_weights[1])[rows] @ x)
        gate = bf16_round(f64(g.gate_proj_weights[1])[rows] @ x)
        want = bf16_round(bf16_round(gate / (1 + np.exp(-gate))) * up)
        got = f64(g.silu_out)[rows]
        assert np.abs(got - want).max() <= BF16_EPS * max(np.abs(want).max(), 1e-3) * 2.1
    assert int(g.barriers[1, 4, 0]) == 3
    g.barriers[1, 5, 0] = g.down_proj_total_jobs()
    pyvm.interpret(g, [RMS_LM_Head(2, 5)])
    x = rms_ref(g.hidden_states, g.lm_head_norm_weights, g.rms_norm_eps)
    want = bf16_round(f64(g.lm_head_weights)[32:80] @ x)
    got = f64(g.logits)[32:80]
    assert np.abs(got - want).max() <= BF16_EPS * np.abs(want).max() * 1.01
    assert (got != want).mean() < 0.1
    assert (f64(g.logits)[:32] == 0).all() and (f64(g.logits)[80:] == 0).all()


# ---------------------------------------------------------------------------------------------
# whole steps
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("cfg,workers,partitions", [
    (config_tiny(), 16, 1), (config_tiny(), 16, 3), (config_1b_slice(), 132, 1), (config_8b_slice(), 256, 2)])
def test_barrier_closed_form_after_a_step(cfg, workers, partitions):
    model, sched, g = fresh(cfg, workers=workers, pos=40, partitions=partitions)
    pyvm.interpret(g, sched.get_linear_instructions())
    H, KVH, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    want = torch.zeros_like(g.barriers)
    want[:, 0, :] = D // 16
    if partitions > 1:
        want[:, 1, :H] = partitions
    want[:, 2, 0] = H
    want[:, 3, 0] = g.o_proj_total_jobs()
    want[:, 4, 0] = cfg.intermediate_size // 16
    want[:, 5, 0] = g.down_proj_total_jobs()
    assert torch.equal(g.barriers, want)


def test_invalid_order_trips_the_barrier_assertions():
    cfg = config_tiny()
    model, sched, g = fresh(cfg)
    ins = sched.get_linear_instructions()
    first_attention = next(i for i, x in enumerate(ins) if x.opcode() == 2)
    with pytest.raises(pyvm.OracleError, match="attention"):
        pyvm.interpret(g, ins[:4] + [ins[first_attention]])
    g.barriers.zero_()
    with pytest.raises(pyvm.OracleError, match="upgate"):
        pyvm.interpret(g, [x for x in ins if x.opcode() != 4][: first_attention + 40])
    g.barriers.zero_()
    # running an instruction twice breaks the exact counts for its successor
    lm = [x for x in ins if x.opcode() == 7][0]
    with pytest.raises(pyvm.OracleError):
        pyvm.interpret(g, ins[:-16] + [ins[-17]] + [lm])
    with pytest.raises(pyvm.OracleError, match="unknown opcode"):
        pyvm.interpret(g, torch.tensor([[9] + [0] * 31], dtype=torch.int32))


@pytest.mark.parametrize("cfg,workers,partitions,pos", [
    (config_tiny(), 16, 1, 37), (config_tiny(), 16, 4, 120), (config_1b_slice(), 148, 1, 90),
    (config_8b_slice(), 256, 1, 45)])
def test_step_matches_torch_restatement(cfg, workers, partitions, pos):
    """C checker vs the restatement written with the reference's torch operations: every buffer
    within bf16 rounding (they differ in fp32 summation order only), barriers identical."""
    model, sched, g = fresh(cfg, workers=workers, pos=pos, partitions=partitions)
    model_t, sched_t, gt = fresh(cfg, workers=workers, pos=pos, partitions=partitions)
    pyvm.interpret(g, sched.get_linear_instructions())
    pyvm_torch.interpret(gt, sched_t.get_linear_instructions())
    assert torch.equal(g.barriers, gt.barriers)
    for name in ("hidden_states", "post_ln_rope_q", "attn_out", "silu_out", "logits"):
        a, b = getattr(g, name).float(), getattr(gt, name).float()
        scale = b.abs().max()
        # stated tolerance: max error <= 2e-2 of the tensor's largest magnitude (a few bf16 ulps
        # after accumulation through the layers); typical error is far below one ulp
        assert (a - b).abs().max() <= 2e-2 * scale, name
        assert (a - b).abs().mean() <= 2e-3 * scale, name
    for cache in ("k_cache", "v_cache"):
        a, b = getattr(g, cache)[:, :, pos].float(), getattr(gt, cache)[:, :, pos].float()
        assert (a - b).abs().max() <= 2e-2 * b.abs().max()
    if partitions > 1:
        a, b = g.attn_out_intermediates[:, :partitions], gt.attn_out_intermediates[:, :partitions]
        assert (a - b).abs().max() <= 2e-2 * b.abs().max()
        assert (g.attn_lse_intermediates[:, :partitions] - gt.attn_lse_intermediates[:, :partitions]).abs().max() <= 1e-2


def test_step_matches_plain_llama_forward():
    """One VM step = one decode step of the dense model (prefill by the plain forward, then the
    next token both ways): same greedy token when the top-2 gap is not a tie, logits within bf16
    tolerance."""
    cfg = config_tiny()
    model = make_model(cfg, max_len=64, seed=3)
    prompt = torch.randint(0, cfg.vocab_size, (1, 12), generator=torch.Generator().manual_seed(1))
    out = model(BatchState(input_ids=prompt, position_ids=torch.arange(12)))
    first = int(out.output_ids[0, -1])
    sched = build_schedule(model, 16)
    oracle_gen = pyvm.OracleGenerator(model, sched)
    kv_snapshot = [c.clone() for c in model.stacked_kv_cache]
    tok_vm = oracle_gen.run(first, 12)
    logits_vm = sched.globs.logits.float().clone()
    for c, snap in zip(model.stacked_kv_cache, kv_snapshot):
        c.copy_(snap)
    dense = model(BatchState(input_ids=torch.tensor([[first]]), position_ids=torch.tensor([12]), seq_len=13))
    h = dense.hidden_states
    from megakernels_amd.llama import rms_norm
    logits_dense = torch.nn.functional.linear(
        rms_norm(h, model.lm_head.input_norm.weight, cfg.rms_norm_eps), model.lm_head.lm_head.weight).float().reshape(-1)
    assert (logits_vm - logits_dense).abs().max() <= 2e-2 * logits_dense.abs().max()
    top2 = logits_dense.topk(2).values
    if float(top2[0] - top2[1]) > 4 * BF16_EPS * float(top2[0].abs()):
        assert tok_vm == int(dense.output_ids.reshape(-1)[0])


def test_greedy_decode_loop_is_deterministic_and_appends_kv():
    cfg = config_tiny()
    model = make_model(cfg, max_len=64, seed=4)
    fill_kv(model, upto=8)
    sched = build_schedule(model, 16)
    gen = pyvm.OracleGenerator(model, sched)
    tokens = torch.zeros(1, 6, dtype=torch.long)
    tokens[0, 0] = 17
    gen.generate(tokens, prompt_len=8, ntok=5, ntok_already_generated=1)
    first = tokens.clone()
    assert int(sched.globs.pos_id) == 12
    fill_kv(model, upto=8)
    tokens[0, 1:] = 0
    gen.generate(tokens, prompt_len=8, ntok=5, ntok_already_generated=1)
    assert torch.equal(tokens, first)
    assert pyvm.argmax_bf16(torch.tensor([1.0, 3.0, 3.0, -1.0], dtype=torch.bfloat16)) == 1  # first maximum

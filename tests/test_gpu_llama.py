"""GPU parity of the decode step (ogm_llama_*, through the C ABI) against the CPU restatement
oracle/llama_ref.py on the same seeded model.  The matmuls inside are bit-exact (tested in
test_gpu_parity.py); the element-wise kernels use tree reductions and the device's exp / sin /
cos, so the bar here is a tolerance: hidden state and logits within 2e-4 of the largest magnitude
(stated in `close`), greedy token equal unless the CPU's top two logits are within that tolerance.
Every decode step holds that bound; there is no looser allowance.

Two roundings inside the step are discontinuous, and an f32 difference in the last bit upstream can
tip either: the f16 rounding of a cache row and the int8 rounding of an activation element in a
quantizer.  `step_both` therefore runs the two sides in lock-step at exactly those points: the
device goes first with its debug capture on; the CPU restatement then checks each cache row it is
about to append against the device's (equal up to one f16 step on a few elements) and each
activation it is about to quantize against the device's int8 values and scales (equal up to one
unit on a few elements, scales to 1e-5), and continues from the device's.  What is compared at the
end is then the arithmetic between those points, free of the two amplifiers."""
import sys
from contextlib import contextmanager

import numpy as np
import pytest

from helpers import IQ4_NL, IQ4_XS, Q2_K, Q3_K, Q4_0, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, synth_weights
from oracle import llama_ref as R

pytestmark = pytest.mark.gpu
f32 = np.float32
TOL = 2e-4


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def be():
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()
    yield b
    b.close()


def close(got, want, what):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    scale = np.abs(want).max() + 1e-30
    err = np.abs(got - want).max() / scale
    assert np.isfinite(got).all(), what
    assert err <= TOL, f"{what}: max error {err:.3e} of the largest magnitude {scale:.3e}"
    return err


PRE_SIZES = {"q_bias": lambda nh, nkv, hd: nh * hd, "k_bias": lambda nh, nkv, hd: nkv * hd,
             "v_bias": lambda nh, nkv, hd: nkv * hd, "q_norm": lambda nh, nkv, hd: hd,
             "k_norm": lambda nh, nkv, hd: hd}


def build(be, *, n_embd, n_head, n_kv, hd, n_ff, n_vocab, n_layer, types, max_ctx, seed, rope_dim=None,
          base=10000.0, pre=(), neox=False, freq_factors=None, attn_norm_scale=1.0, pre_scale=None):
    from orangu_amd import LlamaDecoder, QuantMatrix
    rng = np.random.default_rng(seed)
    tq, tv, tdown, tout = types
    mk = lambda t, i, o, s: (t, synth_weights(t, i, o, seed=s), i, o)
    layers = []
    for l in range(n_layer):
        s = seed * 1000 + 10 * l
        layers.append(R.Layer(mk(tq, n_embd, n_head * hd, s + 1), mk(tq, n_embd, n_kv * hd, s + 2),
                              mk(tv, n_embd, n_kv * hd, s + 3), mk(tq, n_head * hd, n_embd, s + 4),
                              mk(tq, n_embd, n_ff, s + 5), mk(tq, n_embd, n_ff, s + 6),
                              mk(tdown, n_ff, n_embd, s + 7),
                              (attn_norm_scale * (1 + 0.1 * rng.standard_normal(n_embd))).astype(f32),
                              (1 + 0.1 * rng.standard_normal(n_embd)).astype(f32)))
        for name in pre:   # biases of the projections' own size, norm weights around one
            n = PRE_SIZES[name](n_head, n_kv, hd)
            # a bias of the size the synthetic weights of that type give the projection itself
            mag = {Q8_0: 0.2, Q4_K: 30.0, Q6_K: 200.0}.get(tv if name == "v_bias" else tq, 1.0)
            vec = (1 + 0.2 * rng.standard_normal(n)) if name.endswith("norm") else mag * rng.standard_normal(n)
            setattr(layers[-1], name, (vec * (pre_scale or {}).get(name, 1.0)).astype(f32))
    out_norm = (1 + 0.1 * rng.standard_normal(n_embd)).astype(f32)
    output = mk(tout, n_embd, n_vocab, seed * 1000 + 999)
    ref = R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd if rope_dim is None else rope_dim, 1e-5, base,
                  layers, out_norm, output, rope_neox=neox, rope_freq_factors=freq_factors)
    ref.reset()
    qm = lambda w: QuantMatrix(np.ascontiguousarray(w[1]), w[0], w[2], w[3])
    dev = LlamaDecoder(be, n_embd=n_embd, n_head=n_head, n_head_kv=n_kv, head_dim=hd, n_ff=n_ff,
                       n_vocab=n_vocab, max_ctx=max_ctx, rope_dim=rope_dim, rms_eps=1e-5, rope_freq_base=base,
                       rope_neox=neox, rope_freq_factors=freq_factors,
                       layers=[{k: (qm(getattr(L, k)) if k.startswith("w") else getattr(L, k))
                                for k in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down", "attn_norm", "ffn_norm")
                                + tuple(pre)}
                               for L in layers],
                       output_norm=out_norm, output=qm(output))
    return ref, dev, rng


def step_both(ref, dev, x, pos, what, attn_rtol=1e-5):
    """One step on both sides, in lock-step at the two discontinuous roundings (module docstring).
    The device goes first.  The CPU restatement then
      * checks each cache row it is about to append against the device's: equal, or for a few
        elements the neighbouring f16 value (an f32 difference in the last bits can fall either
        side of an f16 rounding boundary), plus 1e-5 of the row's largest magnitude; and
      * checks each activation it is about to quantize (vecdot::quantize_act / quantize_act_k_row)
        against the int8 values and scales the device's producing kernel left: scales within 1e-5,
        values equal except for a few elements one unit apart;
    and continues from the device's row and the device's int8 activation.  attn_rtol: the bound on the
    scales of the attention output (site 4 l + 1) alone -- the restatement adds a softmax's terms one
    after the other in f32 as attention.rs does, the device in trees per chunk, and over thousands of
    cached positions with values of both signs the two sums drift apart by more than 1e-5 of the result."""
    import oracle
    dev.capture_acts(True)
    got_logits, got_tok = dev.decode(x, pos)
    got_hidden = dev.hidden()
    rows = [dev.kv_read(l, pos, 1) for l in range(dev.n_layer)]
    acts = [dev.act(site) for site in range(4 * dev.n_layer + 1)]
    dev.capture_acts(False)

    def hook(li, p, k_row, v_row):
        out = []
        for name, mine, theirs in (("k", k_row, rows[li][0][0]), ("v", v_row, rows[li][1][0])):
            a, b = mine.astype(np.float64), theirs.astype(np.float64)
            ulp = np.spacing(np.maximum(np.abs(mine), np.abs(theirs)).astype(np.float16)).astype(np.float64)
            off = a != b
            rowmax = np.abs(b).max()
            # f32 budget: 1e-5 of the row's largest value (the rotation's cosines and sines are the C library's
            # on both sides, so position adds nothing)
            budget = 1e-5 * rowmax
            assert (np.abs(a - b) <= ulp + budget).all(), \
                f"{what}: layer {li} {name} cache row differs by more than one f16 step and the f32 budget " \
                f"(worst {np.abs(a - b).max():.3g}, allowed {(ulp + budget)[np.abs(a - b).argmax()]:.3g})"
            assert off.mean() <= 0.05, f"{what}: layer {li} {name} cache row: {off.sum()} of {off.size} elements differ"
            out.append(theirs.copy())
        return out

    def act_hook(site, xin, group):
        q_dev, d_dev, g_dev = acts[site]
        assert g_dev == group and q_dev.size == xin.size, f"{what}: site {site}: quantizer group or width"
        q_cpu, d_cpu, _ = (oracle.quantize_act if group == 32 else oracle.quantize_act_k_row)(xin)
        rtol = attn_rtol if site % 4 == 1 else 1e-5
        assert np.allclose(d_dev, d_cpu, rtol=rtol, atol=1e-30), f"{what}: site {site}: activation scales"
        diff = np.abs(q_dev.astype(np.int32) - q_cpu.astype(np.int32))
        n_off = int((diff != 0).sum())
        assert diff.max() <= 1 and n_off <= max(3, q_dev.size // 500, int(q_dev.size * rtol * 100)), \
            f"{what}: site {site}: {n_off} of {q_dev.size} int8 activations differ, by up to {diff.max()}"
        if n_off:
            say(f"{what}: site {site}: {n_off} int8 activation(s) one unit apart; the CPU continues from the device's")
        return q_dev, d_dev

    ref.act_hook = act_hook
    ref.kv_hook = hook
    try:
        want_logits, want_hidden = R.decode_step(ref, x, pos)
    finally:
        ref.kv_hook = None
        ref.act_hook = None
    e1 = close(got_hidden, want_hidden, f"{what}: hidden state")
    e2 = close(got_logits, want_logits, f"{what}: logits")
    top = np.sort(want_logits)[-2:]
    if top[1] - top[0] > TOL * np.abs(want_logits).max():
        assert got_tok == R.argmax(want_logits), f"{what}: greedy token"
    assert got_tok == R.argmax(got_logits), f"{what}: device argmax of its own logits"
    say(what, "hidden err %.2e logits err %.2e token %d" % (e1, e2, got_tok))


@pytest.mark.parametrize("types", [(Q4_K, Q6_K, Q6_K, Q6_K), (Q8_0, Q8_0, Q8_0, Q8_0), (Q4_K, Q4_K, Q4_K, Q4_K),
                                   (Q5_K, Q5_K, Q6_K, Q5_K), (Q4_0, Q5_0, IQ4_NL, Q8_0), (IQ4_XS, Q2_K, IQ4_XS, Q2_K),
                                   (Q5_1, Q5_1, Q5_1, Q5_1)])
def test_decode_steps_from_an_empty_cache(be, types):
    """Positions 0..5 one after the other: RMSNorm, q/k/v, RoPE, cache append, attention over the
    growing cache, wo, residual, SwiGLU FFN, output norm and vocabulary projection."""
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320,
                          n_layer=1 if Q2_K in types else 2, types=types, max_ctx=16, seed=5)
    try:
        for pos in range(6):
            step_both(ref, dev, rng.standard_normal(256).astype(f32), pos, f"types {types} pos {pos}")
    finally:
        dev.close()


def test_decode_with_a_cache_too_long_for_a_table_of_every_position(be):
    """The rotation table of every position is made once at creation while it stays under 64 MiB; a longer
    cache (here 300 000 positions of 32 pairs) computes each token's row when it is decoded.  Same steps."""
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=1, hd=64, n_ff=512, n_vocab=320, n_layer=1,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=300000, seed=8)
    try:
        for pos in range(4):
            step_both(ref, dev, rng.standard_normal(256).astype(f32), pos, f"long cache pos {pos}")
    finally:
        dev.close()


def test_decode_with_q3_k_value_and_down_projections(be):
    """Q3_K in the v and down projections (what a Q3_K_M file does), one layer: the synthetic Q3_K
    weights are large, and with two layers of them the final hidden state is a small difference of
    huge terms whose f16 cache rounding dominates any tolerance relative to the result."""
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=1,
                          types=(Q4_K, Q3_K, Q3_K, Q5_K), max_ctx=16, seed=5)
    try:
        for pos in range(5):
            step_both(ref, dev, rng.standard_normal(256).astype(f32), pos, f"q3_k v/down pos {pos}")
    finally:
        dev.close()


def test_decode_over_a_prefilled_cache_with_several_attention_chunks(be):
    """head_dim 128, four query heads per K/V head, 300 cached positions handed over from the host
    (three attention chunks, the last one partial), partial rotary dimension."""
    n_kv, hd = 2, 128
    ref, dev, rng = build(be, n_embd=1024, n_head=8, n_kv=n_kv, hd=hd, n_ff=2816, n_vocab=1000, n_layer=3,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=512, seed=6, rope_dim=64, base=500000.0)
    try:
        n_pre = 300
        for l in range(3):
            k = rng.standard_normal((n_pre, n_kv * hd)).astype(f32)
            v = rng.standard_normal((n_pre, n_kv * hd)).astype(f32)
            dev.kv_write(l, 0, k, v)
            ref.k_cache[l] = [r.astype(np.float16) for r in k]
            ref.v_cache[l] = [r.astype(np.float16) for r in v]
        for pos in (300, 301, 302):
            step_both(ref, dev, rng.standard_normal(1024).astype(f32), pos, f"prefilled pos {pos}")
    finally:
        dev.close()


@pytest.mark.parametrize("hd,group,n_kv,n_pre", [(128, 4, 1, 4500), (128, 8, 1, 2200), (64, 4, 2, 8300), (128, 1, 2, 16500)])
def test_decode_at_contexts_whose_chunks_merge_in_several_rounds(be, hd, group, n_kv, n_pre):
    """The workgroup that merges a K/V head's chunks takes up to eight chunks per slice in one trip to
    memory (32 chunks at head_dim 128 with four query heads, 16 with eight, 64 at head_dim 64 with four, 128
    with one query head) and goes round again for longer contexts, carrying its running maximum; here 36, 18, 65
    and 129 chunks, the last one partial.  (The attention output's scales differ from the restatement's by up to 1.5e-4
    of their value at these lengths -- its softmax sums run term by term in f32 -- against 1e-2 and more for a chunk left
    out; the bound grows with the context.)"""
    n_head = group * n_kv
    n_embd = 256
    ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=320, n_layer=1,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=n_pre + 4, seed=9, base=500000.0,
                          attn_norm_scale=TAME[Q4_K])   # scores of order one: every chunk carries weight
    try:
        fill_cache_both(ref, dev, rng, 1, n_pre, n_kv * hd)
        for pos in (n_pre, n_pre + 1):
            step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), pos, f"context {pos}", attn_rtol=1e-5 * n_pre / 250)
    finally:
        dev.close()


@pytest.mark.parametrize("hd,group,n_kv,n_pre,chunks", [
    (128, 4, 1, 4500, 3), (128, 8, 1, 2200, 2), (64, 4, 2, 8300, 5), (128, 1, 2, 16500, 16), (128, 4, 2, 300, 2),
    (64, 8, 1, 700, 4), (128, 2, 1, 130, 64), (128, 1, 8, 8300, 0)])
def test_decode_with_several_chunks_per_workgroup(be, hd, group, n_kv, n_pre, chunks):
    """On long contexts a workgroup of the decode step's attention takes several chunks of the cache in a row and
    keeps a running maximum, sum and weighted V sum (by default as many as keep the launch near 512 workgroups:
    two at 8300 positions of eight K/V heads, the last case; forced here otherwise: 2 to 16 chunks, more than the
    context has, chunks of 64 positions, two outputs per thread at eight query heads).  Same allowances as with a
    chunk per workgroup."""
    n_head = group * n_kv
    n_embd = 256
    ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=320, n_layer=1,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=n_pre + 4, seed=19, base=500000.0,
                          attn_norm_scale=TAME[Q4_K])
    be.set_tuning("attn_decode_chunks", chunks)
    try:
        fill_cache_both(ref, dev, rng, 1, n_pre, n_kv * hd)
        for pos in (n_pre, n_pre + 1):
            step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), pos, f"context {pos}, {chunks} chunks a workgroup",
                      attn_rtol=1e-5 * max(n_pre, 250) / 250)
    finally:
        be.set_tuning("attn_decode_chunks", 0)
        dev.close()


@contextmanager
def llama_8b_prefix(be, ctx, dims=(4096, 32, 8, 128, 14336, 128256), n_layer=2):
    """A two-layer prefix of the 8B-shaped Q4_K_M-like model (hidden 4096, 32 query heads over 8 K/V heads
    of 128, FFN 14336 with a Q6_K down projection, the Q6_K 128256-row output, RoPE base 500000) on both
    sides, over an f16 cache holding `ctx` random positions.  Yields (ref, dev, rng).  dims: another model's
    (n_embd, n_head, n_kv, head_dim, n_ff, n_vocab) with the same matrix types."""
    n_embd, n_head, n_kv, hd, n_ff, n_vocab = dims
    from orangu_amd import LlamaDecoder, QuantMatrix
    rng = np.random.default_rng(515)
    shapes = {"wq": (Q4_K, n_embd, n_embd), "wk": (Q4_K, n_embd, n_kv * hd), "wv": (Q4_K, n_embd, n_kv * hd),
              "wo": (Q4_K, n_embd, n_embd), "w_gate": (Q4_K, n_embd, n_ff), "w_up": (Q4_K, n_embd, n_ff),
              "w_down": (Q6_K, n_ff, n_embd)}
    order = ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")
    ref_layers, dev_layers = [], []
    for l in range(n_layer):
        w = {k: (t, synth_weights(t, i, o, seed=600 + 10 * l + n), i, o) for n, (k, (t, i, o)) in enumerate(shapes.items())}
        norms = [(1 + 0.05 * rng.standard_normal(n_embd)).astype(f32) for _ in range(2)]
        ref_layers.append(R.Layer(*[w[k] for k in order], *norms))
        dev_layers.append({**{k: QuantMatrix(w[k][1], w[k][0], w[k][2], w[k][3]) for k in order},
                           "attn_norm": norms[0], "ffn_norm": norms[1]})
    out_norm = (1 + 0.05 * rng.standard_normal(n_embd)).astype(f32)
    out = (Q6_K, synth_weights(Q6_K, n_embd, n_vocab, seed=699), n_embd, n_vocab)
    ref = R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd, 1e-5, 500000.0, ref_layers, out_norm, out)
    ref.reset()
    out_qm = QuantMatrix(out[1], out[0], out[2], out[3])
    dev = LlamaDecoder(be, n_embd=n_embd, n_head=n_head, n_head_kv=n_kv, head_dim=hd, n_ff=n_ff, n_vocab=n_vocab,
                       max_ctx=ctx + 16, rms_eps=1e-5, rope_freq_base=500000.0, layers=dev_layers,
                       output_norm=out_norm, output=out_qm)
    try:
        for l in range(n_layer):
            k = rng.standard_normal((ctx, n_kv * hd)).astype(f32)
            v = rng.standard_normal((ctx, n_kv * hd)).astype(f32)
            dev.kv_write(l, 0, k, v)
            ref.k_cache[l] = [r.astype(np.float16) for r in k]
            ref.v_cache[l] = [r.astype(np.float16) for r in v]
        yield ref, dev, rng
    finally:
        dev.close()
        for L in dev_layers:   # 0.9 GB of weights: give them back before the next test
            for k in order:
                be.evict(L[k])
        be.evict(out_qm)


def test_llama_8b_shaped_layers_at_context_2048(be):
    """Config 5 at its real shapes: two decode steps of the two-layer 8B prefix at context 2048 against
    the CPU restatement."""
    ctx = 2048
    with llama_8b_prefix(be, ctx) as (ref, dev, rng):
        for pos in (ctx, ctx + 1):
            step_both(ref, dev, rng.standard_normal(4096).astype(f32), pos, f"8B shapes pos {pos}")


def test_llama_405b_shaped_layer(be):
    """One layer at Llama-3.1-405B's shapes (hidden 16384, 128 query heads over 8 K/V heads of 128 -- sixteen to a
    K/V head, two workgroups of eight in the attention kernel --, FFN 53248; 1.9 GB of Q4_K / Q6_K weights, a
    1024-row output matrix) over 300 cached positions: two decode steps and a verify batch of four against the CPU
    restatement.  The whole model in this quantization is 230 GB: one MI355X holds it."""
    ctx = 300
    with llama_8b_prefix(be, ctx, dims=(16384, 128, 8, 128, 53248, 1024), n_layer=1) as (ref, dev, rng):
        for pos in (ctx, ctx + 1):
            step_both(ref, dev, rng.standard_normal(16384).astype(f32), pos, f"405B shapes pos {pos}")
        prefill_both(ref, dev, rng.standard_normal((4, 16384)).astype(f32), ctx + 2, "405B shapes, verify batch of 4")


def test_llama_8b_shaped_verify_batches_at_context_2048(be):
    """The speculative-decode verify shape (generate.rs:1618-1674: the last accepted token plus the draft
    go through the model as one batch, matmuls at n_tokens = 1 + draft, cpu.rs:265-317) at the 8B shapes:
    batches of 4 and then 8 tokens appended at position 2048 of the two-layer prefix, against the CPU
    restatement -- the first through forward_all_logits (every position's logits and greedy token: what the
    verify step compares the draft with), the second through the prefill entry (the last position's).  The second batch starts where the first did, as after a draft that was rejected whole:
    both sides drop the first batch's cache rows."""
    ctx = 2048
    with llama_8b_prefix(be, ctx) as (ref, dev, rng):
        for n_tokens in (4, 8):
            for l in range(2):
                del ref.k_cache[l][ctx:], ref.v_cache[l][ctx:]
            X = rng.standard_normal((n_tokens, 4096)).astype(f32)
            prefill_both(ref, dev, X, ctx, f"8B shapes, verify batch of {n_tokens}", all_logits=n_tokens == 4)
        # the step after an accepted batch continues on the rows the batch wrote
        step_both(ref, dev, rng.standard_normal(4096).astype(f32), ctx + 8, "8B shapes, step after the verify batch")


def test_cache_rows_beyond_the_f16_range_saturate(be):
    """K/V components beyond +-65504 are cached as +-65504, not as infinities: rows handed over from
    the host and rows the decode step writes itself (a v bias of 1e5), and the step after them stays
    finite and agrees with the CPU restatement, whose f16 cache saturates the same way."""
    n_kv, hd = 2, 64
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=300, n_layer=2,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=16, seed=77, pre=("v_bias",),
                          pre_scale={"v_bias": 500.0})
    try:
        k = rng.standard_normal((3, n_kv * hd)).astype(f32)
        v = rng.standard_normal((3, n_kv * hd)).astype(f32)
        v[1, 7], v[2, 9], k[0, 3] = 1.0e6, -7.0e4, 65519.0
        for l in range(2):
            dev.kv_write(l, 0, k, v)
            ref.k_cache[l] = [R.to_cache(r, np.float16) for r in k]
            ref.v_cache[l] = [R.to_cache(r, np.float16) for r in v]
        kb, vb = dev.kv_read(0, 0, 3)
        assert vb.view(np.uint16)[1, 7] == 0x7BFF and vb.view(np.uint16)[2, 9] == 0xFBFF and kb.view(np.uint16)[0, 3] == 0x7BFF
        for pos in (3, 4):
            step_both(ref, dev, rng.standard_normal(256).astype(f32), pos, f"saturated cache pos {pos}")
        _, vb = dev.kv_read(1, 3, 2)
        assert np.isfinite(vb.astype(f32)).all()
        assert (np.abs(vb.astype(f32)) == 65504.0).any(), "the bias was meant to push some v components out of range"
    finally:
        dev.close()


@pytest.mark.parametrize("hd,group,n_kv", [(128, 1, 2), (128, 2, 2), (128, 8, 1), (64, 1, 4), (64, 4, 2), (64, 8, 1)])
@pytest.mark.parametrize("wtype", [Q4_K, Q8_0])
def test_attention_head_shapes_across_a_chunk_boundary(be, hd, group, n_kv, wtype):
    """Every (head_dim, query heads per K/V head) the attention kernel is built for, with per-256
    and per-32 quantization of its output, over positions 126..130: the last row of a full chunk,
    then a chunk that holds the current position only."""
    n_head = group * n_kv
    n_embd = n_head * hd
    ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=256, n_layer=2,
                          types=(wtype, wtype, wtype, wtype), max_ctx=160, seed=hd + group, rope_dim=hd // 2)
    try:
        n_pre = 126
        for l in range(2):
            k = rng.standard_normal((n_pre, n_kv * hd)).astype(f32)
            v = rng.standard_normal((n_pre, n_kv * hd)).astype(f32)
            dev.kv_write(l, 0, k, v)
            ref.k_cache[l] = [r.astype(np.float16) for r in k]
            ref.v_cache[l] = [r.astype(np.float16) for r in v]
        for pos in range(126, 131):
            step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), pos, f"hd {hd} group {group} pos {pos}")
    finally:
        dev.close()


def fill_cache_both(ref, dev, rng, n_layer, n_pre, kv_dim):
    for l in range(n_layer):
        k = rng.standard_normal((n_pre, kv_dim)).astype(f32)
        v = rng.standard_normal((n_pre, kv_dim)).astype(f32)
        dev.kv_write(l, 0, k, v)
        ref.k_cache[l] = [r.astype(np.float16) for r in k]
        ref.v_cache[l] = [r.astype(np.float16) for r in v]


@pytest.mark.parametrize("hd,group,n_kv", [(128, 3, 2), (128, 5, 2), (128, 6, 1), (128, 7, 2), (64, 3, 4), (64, 7, 4)])
@pytest.mark.parametrize("wtype", [Q4_K, Q8_0])
def test_attention_with_odd_query_groups(be, hd, group, n_kv, wtype):
    """Query heads per K/V head that are not a power of two (Llama-3.2-3B has 3, Qwen2.5-7B has 7):
    the kernel runs with the next power of two of head slots, the spare ones empty."""
    n_head = group * n_kv
    n_embd = n_head * hd
    ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=256, n_layer=2,
                          types=(wtype, wtype, wtype, wtype), max_ctx=160, seed=3 * hd + group)
    try:
        fill_cache_both(ref, dev, rng, 2, 127, n_kv * hd)
        for pos in range(127, 130):
            step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), pos, f"hd {hd} group {group} pos {pos}")
    finally:
        dev.close()


@pytest.mark.parametrize("hd,group,n_kv", [(128, 16, 1), (64, 12, 2), (128, 10, 1), (64, 24, 1)])
def test_attention_with_more_than_eight_query_heads_per_kv_head(be, hd, group, n_kv):
    """Llama-3.1-405B has 16 query heads per K/V head, Mistral-Large-2 has 12: the attention kernels deal such a
    group to workgroups in equal parts of at most eight heads (16 = 2 x 8, 12 = 2 x 6, 10 = 2 x 5, 24 = 3 x 8).
    Decode steps across a chunk boundary, then prefills on both prefill attention kernels and a verify batch; a
    count that does not divide (9) is refused at creation."""
    from orangu_amd import LlamaDecoder, OgmError
    n_head = group * n_kv
    n_embd = n_head * hd
    ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=256, n_layer=2,
                          types=(Q4_K, Q4_K, Q6_K, Q6_K), max_ctx=200, seed=5 * hd + group, attn_norm_scale=TAME[Q4_K])
    try:
        fill_cache_both(ref, dev, rng, 2, 127, n_kv * hd)
        for pos in range(127, 130):
            step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), pos, f"hd {hd} group {group} pos {pos}")
        for variant, T in ((1, 5), (2, 40), (0, 60)):
            be.set_tuning("attn_prefill_variant", variant)
            ref.reset()
            prefill_both(ref, dev, rng.standard_normal((T, n_embd)).astype(f32), 0, f"group {group}, prefill of {T}, variant {variant}")
        # (rows of their own seed: with the stream's next rows the 10-head model rounds one last-layer activation the
        # other way on the device, which no cache row shows and moves the logits by 6e-4)
        xv = np.random.default_rng(1234 + group).standard_normal((4, n_embd)).astype(f32)
        prefill_both(ref, dev, xv, 60, f"group {group}, verify batch")
    finally:
        be.set_tuning("attn_prefill_variant", 0)
        dev.close()
    if group == 16:
        with pytest.raises(OgmError):
            build(be, n_embd=9 * 64, n_head=9, n_kv=1, hd=64, n_ff=512, n_vocab=256, n_layer=1,
                  types=(Q8_0, Q8_0, Q8_0, Q8_0), max_ctx=8, seed=1)


@pytest.mark.parametrize("pre,neox,ff,rope_dim", [
    ((), True, False, None),                                       # NEOX pairing alone
    ((), True, False, 32),                                         # NEOX over part of the head
    ((), False, True, None),                                       # Llama-3.1: frequency factors, NORM pairs
    (("q_bias", "k_bias", "v_bias"), True, False, None),           # Qwen2
    (("q_norm", "k_norm"), True, False, None),                     # Qwen3
    (("q_bias", "k_bias", "v_bias", "q_norm", "k_norm"), True, True, 32),
    (("v_bias", "q_norm"), False, True, None),                     # each tensor is optional on its own
])
@pytest.mark.parametrize("hd,group,n_kv,wtype", [(128, 4, 2, Q4_K), (64, 7, 4, Q8_0), (64, 2, 2, Q6_K)])
def test_bias_head_norm_pairing_and_frequency_factors(be, pre, neox, ff, rope_dim, hd, group, n_kv, wtype):
    """What llama.rs:757-810 applies between the projections and the attention, for the files its
    loader routes there: bias, then per-head RMSNorm of q and k, then RoPE in the file's pairing
    with rope_freqs.weight dividing the frequencies.  From an empty cache (the rows written are
    the rotated ones) and across a chunk boundary of a prefilled one."""
    n_head = group * n_kv
    n_embd = n_head * hd
    rd = hd if rope_dim is None else rope_dim
    factors = np.linspace(1.0, 8.0, rd // 2).astype(f32) if ff else None
    kw = dict(n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=256, n_layer=2,
              types=(wtype, wtype, wtype, wtype), max_ctx=160, seed=hd + 7 * group + len(pre), rope_dim=rope_dim,
              pre=pre, neox=neox, freq_factors=factors)
    ref, dev, rng = build(be, **kw)
    try:
        for pos in range(4):
            step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), pos, f"{pre} neox {neox} ff {ff} pos {pos}")
    finally:
        dev.close()
    ref, dev, rng = build(be, **kw)
    try:
        fill_cache_both(ref, dev, rng, 2, 127, n_kv * hd)
        for pos in (127, 128):
            step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), pos, f"{pre} neox {neox} ff {ff} pos {pos}")
    finally:
        dev.close()


def test_decode_rejects_bad_arguments(be):
    from orangu_amd import OgmError
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=1,
                          types=(Q4_K, Q4_K, Q4_K, Q4_K), max_ctx=4, seed=7)
    try:
        with pytest.raises(OgmError):
            dev.decode(np.zeros(256, f32), 4)          # beyond the cache
        with pytest.raises(ValueError):
            dev.decode(np.zeros(100, f32), 0)
        with pytest.raises(OgmError):
            dev.kv_write(0, 3, np.zeros((2, 128), f32), np.zeros((2, 128), f32))
    finally:
        dev.close()


def test_matrices_uploaded_from_a_gguf_file_multiply_like_direct_uploads(be, tmp_path):
    """GGUF reader -> uploader: the same bytes reach the device as through QuantMatrix."""
    import oracle
    from orangu_amd import QuantMatrix
    from orangu_amd.gguf import GgufFile
    from orangu_amd.hiprt import DeviceBuffer, device_synchronize
    from test_gguf_cpu import gguf, gstr, kv, tensor_info
    specs = [("blk.0.ffn_gate.weight", Q4_K, 512, 70), ("blk.0.ffn_down.weight", Q6_K, 256, 33),
             ("blk.0.attn_q.weight", Q8_0, 96, 17)]
    blobs, infos, pos = [], [], 0
    for i, (name, t, n_in, n_out) in enumerate(specs):
        w = synth_weights(t, n_in, n_out, seed=20 + i)
        infos.append(tensor_info(name, [n_in, n_out], t, pos))
        blobs.append(w.tobytes() + b"\0" * ((-w.size) % 32))
        pos += len(blobs[-1])
    b, _ = gguf([kv("general.architecture", 8, gstr("llama"))], infos, data=b"".join(blobs))
    path = tmp_path / "tiny.gguf"
    path.write_bytes(b)
    g = GgufFile(str(path))
    for name, t, n_in, n_out in specs:
        h = g.upload_matrix(be, name)
        assert g.upload_matrix(be, name) == h          # same bytes, same key: one device copy
        x = np.random.default_rng(n_in).standard_normal(n_in).astype(f32)
        xd, yd = DeviceBuffer.from_numpy(x), DeviceBuffer(4 * n_out)
        be.matmul_dev(h, xd.ptr, 1, yd.ptr)
        device_synchronize()
        raw = g.matrix(name)[4]
        want = oracle.matmul(t, raw, n_in, n_out, x, 1).reshape(-1)
        got = yd.to_numpy(f32, n_out)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name
        assert np.array_equal(got, be.matmul(x, 1, QuantMatrix(raw, t, n_in, n_out)))
        xd.free()
        yd.free()
    g.close()


# The synthetic K-quant weights give projections of magnitude 30 to 200 and with them attention
# scores in the thousands: a softmax that picks one position, discontinuously.  Small attention
# norm weights bring the scores of the batch tests to order one.
TAME = {Q4_K: 0.02, Q5_K: 0.02, Q4_0: 0.1}


def prefill_both(ref, dev, X, pos0, what, via_tokens=None, all_logits=False):
    """A batch of tokens on both sides, cache rows in lock-step as in `step_both`.  A flipped
    activation rounding touches one token's rows from the next layer on.  Measured on 600 tokens of
    the two-layer test model: about 50 such events (3e-5 per rounded element), each confined to one
    token, moving its next rows by 1e-4 .. 2e-2 of their largest value (one quantizer step of one
    activation times a column of the synthetic weights; over 1100 tokens the largest seen is 6e-2).
    So up to 1 + T/8 tokens may be off the tight bound, by up to 0.2, and the last token's outputs
    are compared loosely when it is among them; an error of the code would show on every token, or
    be of order one.  All other tokens' rows match to 1e-5 plus one f16 step.
    all_logits: through forward_all_logits instead -- every position's logits and greedy token."""
    T = X.shape[0]
    if all_logits:
        got_all, got_toks = dev.forward_all_logits(X, pos0) if via_tokens is None else \
            dev.forward_all_logits(None, pos0, tok_embd=via_tokens[0], tokens=via_tokens[1])
    else:
        got_logits, got_tok = dev.prefill(X, pos0) if via_tokens is None else dev.prefill_tokens(via_tokens[0], via_tokens[1], pos0)
        got_hidden = dev.hidden()
    rows = [dev.kv_read(l, pos0, T) for l in range(dev.n_layer)]
    flagged = set()

    def hook(li, p, k_row, v_row):
        out = []
        for name, mine, theirs in (("k", k_row, rows[li][0][p - pos0]), ("v", v_row, rows[li][1][p - pos0])):
            a, b = mine.astype(np.float64), theirs.astype(np.float64)
            ulp = np.spacing(np.maximum(np.abs(mine), np.abs(theirs)).astype(np.float16)).astype(np.float64)
            rowmax = np.abs(b).max()
            if not (np.abs(a - b) <= ulp + 1e-5 * rowmax).all():
                assert (np.abs(a - b) <= ulp + 0.2 * rowmax).all(), \
                    f"{what}: position {p} layer {li} {name} cache row differs by more than one f16 step and the f32 budget"
                flagged.add(p)
            out.append(theirs.copy())
        return out

    ref.kv_hook = hook
    if all_logits:
        want_all, _ = R.forward(ref, X, pos0, all_logits=True)
        ref.kv_hook = None
        assert len(flagged) <= 1 + T // 8, f"{what}: {len(flagged)} of {T} tokens off the tight bound: {sorted(flagged)}"
        want_all = np.asarray(want_all, np.float64).reshape(T, -1)
        for t in range(T):
            tol = 0.2 if pos0 + t in flagged else TOL
            err = np.abs(got_all[t].astype(np.float64) - want_all[t]).max() / (np.abs(want_all[t]).max() + 1e-30)
            assert np.isfinite(got_all[t]).all() and err <= tol, f"{what}: logits of position {pos0 + t}: max error {err:.3e}"
            top = np.sort(want_all[t])[-2:]
            if top[1] - top[0] > tol * np.abs(want_all[t]).max():
                assert int(got_toks[t]) == R.argmax(want_all[t]), f"{what}: greedy token of position {pos0 + t}"
            assert int(got_toks[t]) == R.argmax(got_all[t]), f"{what}: device argmax of its own logits, position {pos0 + t}"
        say(what, f"{T} positions from {pos0}: flagged {sorted(flagged)}, tokens {[int(v) for v in got_toks]}")
        return
    want_logits, want_hidden = R.forward(ref, X, pos0)
    ref.kv_hook = None
    assert len(flagged) <= 1 + T // 8, f"{what}: {len(flagged)} of {T} tokens off the tight bound: {sorted(flagged)}"
    tol = 0.2 if pos0 + T - 1 in flagged else TOL
    for name, got, want in (("hidden state", got_hidden, want_hidden), ("logits", got_logits, want_logits)):
        err = np.abs(np.asarray(got, np.float64) - want).max() / (np.abs(want).max() + 1e-30)
        assert np.isfinite(got).all() and err <= tol, f"{what}: {name}: max error {err:.3e}"
    top = np.sort(want_logits)[-2:]
    if top[1] - top[0] > tol * np.abs(want_logits).max():
        assert got_tok == R.argmax(want_logits), f"{what}: greedy token"
    say(what, f"{T} tokens from {pos0}: flagged {sorted(flagged)}, token {got_tok}")


@pytest.mark.parametrize("types", [(Q4_K, Q6_K, Q6_K, Q6_K), (Q8_0, Q8_0, Q8_0, Q8_0), (Q5_K, Q3_K, Q6_K, Q5_K),
                                   (Q4_0, Q5_0, IQ4_NL, Q8_0), (IQ4_XS, Q2_K, IQ4_XS, Q2_K), (Q5_1, Q5_1, Q5_1, Q5_1)])
@pytest.mark.parametrize("n_tokens", [2, 7, 40])
def test_prefill_from_an_empty_cache_then_decode(be, types, n_tokens):
    """run_layers at n_tokens > 1 (llama.rs:594-932): 2 and 7 tokens take the multi-token GEMV in
    the GEMM's float order, 40 the MFMA GEMMs; the decode steps after it continue on the cache the
    prefill wrote."""
    n_layer = 1 if Q3_K in types or Q2_K in types else 2    # two layers of the large synthetic Q3_K / Q2_K weights cancel badly
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=n_layer,
                          types=types, max_ctx=64, seed=51, attn_norm_scale=TAME.get(types[0], 1.0))
    try:
        prefill_both(ref, dev, rng.standard_normal((n_tokens, 256)).astype(f32), 0, f"types {types}")
        for pos in (n_tokens, n_tokens + 1):
            step_both(ref, dev, rng.standard_normal(256).astype(f32), pos, f"types {types} then pos {pos}")
    finally:
        dev.close()


@pytest.mark.parametrize("interleave,n_tokens", [(1, 45), (2, 45), (1, 300), (2, 300), (2, 129)])
def test_prefill_through_the_plane_kernels(be, interleave, n_tokens):
    """The tiled GEMMs over prebuilt planes, forced on a small model (gemm_plane_kernel 2): the norm and SwiGLU
    kernels then write the GEMMs' operand chunks themselves, here with a last token block of 13, 12 and 1 tokens
    (the block's other places keep whatever the buffer held: multiplied, never stored), read by the 128-row kernel
    (gemm_interleave 1) and by the 64-row one (2).  Checked like every prefill, and the matmuls' names."""
    be.set_tuning("gemm_plane_kernel", 2)
    be.set_tuning("gemm_interleave", interleave)
    be.set_tuning("gemm_small_max_tokens", 1)
    be.set_tuning("gemm_medium", 1)
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=2,
                          types=(Q4_K, Q6_K, Q6_K, Q5_K), max_ctx=320, seed=57, attn_norm_scale=TAME[Q4_K])
    try:
        # a longer batch first, so that the chunks of the ragged batch hold another batch's tokens past its last
        dev.prefill(rng.standard_normal((min(320, n_tokens + 19), 256)).astype(f32), 0)
        prefill_both(ref, dev, rng.standard_normal((n_tokens, 256)).astype(f32), 0, f"plane kernels, interleave {interleave}")
        # (under these settings a matmul of the model's shapes takes the kernel meant)
        from orangu_amd import QuantMatrix
        L0 = ref.layers[0].w_gate
        be.matmul(rng.standard_normal(n_tokens * 256).astype(f32), n_tokens, QuantMatrix(np.ascontiguousarray(L0[1]), L0[0], L0[2], L0[3]))
        assert be.last_kernel() == ("ogm_gemm_q4k_dmx_kernel" if interleave == 2 else "ogm_gemm_q4k_dma_kernel")
    finally:
        be.set_tuning("gemm_plane_kernel", 0)
        be.set_tuning("gemm_interleave", 0)
        be.set_tuning("gemm_small_max_tokens", 0)
        be.set_tuning("gemm_medium", 0)
        dev.close()


def test_prefill_of_one_token_is_a_decode_step(be):
    """n_tokens == 1 through the batch entry point: the single-token kernels' float order
    (Backend::matmul at one token, cpu.rs:445-458), the same cache row and logits as the step."""
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=2,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=8, seed=81)
    ref2, dev2, _ = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=2,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=8, seed=81)
    try:
        for pos in range(3):
            x = rng.standard_normal(256).astype(f32)
            step_both(ref, dev, x, pos, f"step pos {pos}")
            lg_step, tok_step = dev.decode(x, pos)      # the same step again: same cache row, same logits
            lg_batch, tok_batch = dev2.prefill(x[None, :], pos)
            close(lg_batch, lg_step, f"one-token prefill pos {pos}")
            for l in range(2):
                ks, vs = dev.kv_read(l, pos, 1)
                kb, vb = dev2.kv_read(l, pos, 1)
                assert np.abs(ks.astype(f32) - kb.astype(f32)).max() <= 2e-3 * np.abs(ks.astype(f32)).max()
                assert np.abs(vs.astype(f32) - vb.astype(f32)).max() <= 2e-3 * np.abs(vs.astype(f32)).max()
        prefill_both(ref, dev, rng.standard_normal((1, 256)).astype(f32), 3, "one token as a batch")
    finally:
        dev.close()
        dev2.close()


@pytest.mark.parametrize("hd,group,n_kv,pre,neox,ff", [
    (128, 4, 2, (), False, True),
    (128, 3, 2, ("q_bias", "k_bias", "v_bias"), True, False),
    (64, 7, 4, ("q_norm", "k_norm"), True, False),
    (64, 8, 1, ("q_bias", "k_norm"), False, True),
])
def test_prefill_across_attention_chunks_and_in_two_parts(be, hd, group, n_kv, pre, neox, ff):
    """A prompt in two calls (100 tokens, then 60 that cross position 128), each token attending to
    the chunks its position has, with every option of the projections' post-processing."""
    n_head = group * n_kv
    n_embd = n_head * hd
    factors = np.linspace(1.0, 8.0, hd // 4).astype(f32) if ff else None
    wtype = Q4_K if n_embd % 256 == 0 else Q8_0
    ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=256, n_layer=2,
                          types=(wtype, wtype, wtype, wtype), max_ctx=192, seed=61 + group, rope_dim=hd // 2,
                          pre=pre, neox=neox, freq_factors=factors, attn_norm_scale=TAME.get(wtype, 1.0))
    try:
        prefill_both(ref, dev, rng.standard_normal((100, n_embd)).astype(f32), 0, f"hd {hd} group {group} part 1")
        prefill_both(ref, dev, rng.standard_normal((60, n_embd)).astype(f32), 100, f"hd {hd} group {group} part 2")
        step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), 160, f"hd {hd} group {group} then pos 160")
    finally:
        dev.close()


def test_prefill_longer_than_one_pass_and_from_token_ids(be):
    """1100 tokens run as two passes over the layers (1024 + 76, with the pass size set to 1024; it is fixed
    at a model's first prefill); from token ids the embedding rows are dequantized on the device
    (llama.rs:609-614) and give the same bits as rows passed in."""
    import oracle
    from orangu_amd import QuantMatrix
    be.set_tuning("prefill_chunk_tokens", 1024)
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=2,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=1152, seed=71, attn_norm_scale=TAME[Q4_K])
    embd_raw = synth_weights(Q6_K, 256, 320, seed=72)
    table = oracle.dequantize(Q6_K, embd_raw, 320 * 256).reshape(320, 256)
    tokens = rng.integers(0, 320, 1100).astype(np.uint32)
    try:
        prefill_both(ref, dev, table[tokens], 0, "1100 tokens by id", via_tokens=(QuantMatrix(embd_raw, Q6_K, 256, 320), tokens))
        lg_ids = dev.prefill_tokens(QuantMatrix(embd_raw, Q6_K, 256, 320), tokens[:40], 0)[0]
        lg_rows = dev.prefill(table[tokens[:40]], 0)[0]
        assert np.array_equal(lg_ids.view(np.uint32), lg_rows.view(np.uint32))
        from orangu_amd import OgmError
        with pytest.raises(OgmError):
            dev.prefill(table[tokens[:100]], 1100)           # beyond the cache
        with pytest.raises(OgmError):
            dev.prefill_tokens(QuantMatrix(embd_raw, Q6_K, 256, 320), np.array([5, 320], np.uint32), 0)   # no such token
    finally:
        be.set_tuning("prefill_chunk_tokens", 2048)
        dev.close()


@pytest.mark.parametrize("n_tokens", [1, 7, 40, 300])
def test_hidden_states_of_every_token(be, n_tokens):
    """forward_hidden_states (llama.rs:1034-1045): every token's final hidden state after the output norm,
    from position 0 whatever the cache held, against the CPU restatement in lock-step on the cache rows
    (see prefill_both: an activation rounding that flips moves one token's later rows; here it can also
    flip in the last layer, where no cache row shows it); from token ids the same bits as from rows."""
    import oracle
    from orangu_amd import OgmError, QuantMatrix
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=2,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=320, seed=81, attn_norm_scale=TAME[Q4_K])
    embd_raw = synth_weights(Q6_K, 256, 320, seed=82)
    table = oracle.dequantize(Q6_K, embd_raw, 320 * 256).reshape(320, 256)
    tokens = rng.integers(0, 320, n_tokens).astype(np.uint32)
    X = np.ascontiguousarray(table[tokens])
    T = n_tokens
    try:
        dev.prefill(rng.standard_normal((5, 256)).astype(f32), 0)    # a cache the call must not continue
        got = dev.hidden_states(X)
        assert got.shape == (T, 256) and np.isfinite(got).all()
        rows = [dev.kv_read(l, 0, T) for l in range(dev.n_layer)]
        flagged = set()

        def hook(li, p, k_row, v_row):
            out = []
            for mine, theirs in ((k_row, rows[li][0][p]), (v_row, rows[li][1][p])):
                a, b = mine.astype(np.float64), theirs.astype(np.float64)
                ulp = np.spacing(np.maximum(np.abs(mine), np.abs(theirs)).astype(np.float16)).astype(np.float64)
                rowmax = np.abs(b).max()
                if not (np.abs(a - b) <= ulp + 1e-5 * rowmax).all():
                    assert (np.abs(a - b) <= ulp + 0.2 * rowmax).all(), f"position {p} layer {li}: cache row"
                    flagged.add(p)
                out.append(theirs.copy())
            return out

        ref.kv_hook = hook
        want = R.hidden_states(ref, X)
        ref.kv_hook = None
        err = np.abs(got.astype(np.float64) - want).max(axis=1) / (np.abs(want).max(axis=1) + 1e-30)
        loose = set(np.nonzero(err > TOL)[0].tolist())
        assert err.max() <= 0.2, f"row {int(err.argmax())}: {err.max():.3e}"
        assert len(loose | flagged) <= 1 + T // 8, f"{len(loose | flagged)} of {T} rows off the tight bound"
        say(f"hidden states of {T} tokens: flagged {sorted(flagged)}, loose {sorted(loose)}, max {err.max():.2e}")
        by_id = dev.hidden_states(tok_embd=QuantMatrix(embd_raw, Q6_K, 256, 320), tokens=tokens)
        assert np.array_equal(by_id.view(np.uint32), got.view(np.uint32))
        with pytest.raises(ValueError):
            dev.hidden_states()
        with pytest.raises(OgmError):
            dev.hidden_states(rng.standard_normal((321, 256)).astype(f32))   # beyond the cache
        with pytest.raises(OgmError):
            dev.hidden_states(tok_embd=QuantMatrix(embd_raw, Q6_K, 256, 320), tokens=np.array([320], np.uint32))
    finally:
        dev.close()


@pytest.mark.parametrize("types", [(Q4_K, Q6_K, Q6_K, Q6_K), (Q8_0, Q8_0, Q8_0, Q8_0), (Q5_K, Q5_K, Q6_K, Q5_K)])
@pytest.mark.parametrize("n_draft", [1, 4, 8, 20])
def test_forward_all_logits_of_a_verify_batch(be, types, n_draft):
    """forward_all_logits (arch/mod.rs:2110-2132; speculative_next, generate.rs:1618-1674): a prompt, then the last
    accepted token plus a draft as one batch; the logits and the greedy token of EVERY position against the CPU
    restatement; then the draft is rejected from its second token on and the next batch overwrites those rows."""
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=2,
                          types=types, max_ctx=96, seed=61, attn_norm_scale=TAME.get(types[0], 1.0))
    try:
        prefill_both(ref, dev, rng.standard_normal((30, 256)).astype(f32), 0, f"types {types} prompt")
        X = rng.standard_normal((1 + n_draft, 256)).astype(f32)
        prefill_both(ref, dev, X, 30, f"types {types} verify {1 + n_draft}", all_logits=True)
        for l in range(dev.n_layer):   # accept one drafted token: positions 30, 31 stay
            del ref.k_cache[l][32:], ref.v_cache[l][32:]
        prefill_both(ref, dev, rng.standard_normal((3, 256)).astype(f32), 32, f"types {types} next batch", all_logits=True)
        step_both(ref, dev, rng.standard_normal(256).astype(f32), 35, f"types {types} then a decode step")
    finally:
        dev.close()


def test_forward_all_logits_from_token_ids_and_limits(be):
    """The same from token ids (the embedding rows dequantized on the device), and the call's limits."""
    import oracle
    from orangu_amd import OgmError, QuantMatrix
    ref, dev, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=1,
                          types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=80, seed=62, attn_norm_scale=TAME[Q4_K])
    try:
        emb_raw = synth_weights(Q8_0, 256, 320, seed=63)
        emb = QuantMatrix(emb_raw, Q8_0, 256, 320)
        table = oracle.dequantize(Q8_0, emb_raw, 320 * 256).reshape(320, 256)
        tokens = rng.integers(0, 320, 6).astype(np.uint32)
        prefill_both(ref, dev, table[tokens], 0, "token ids", via_tokens=(emb, tokens), all_logits=True)
        with pytest.raises(OgmError):
            dev.forward_all_logits(rng.standard_normal((65, 256)).astype(f32), 0)        # more than 64 positions
        with pytest.raises(OgmError):
            dev.forward_all_logits(rng.standard_normal((10, 256)).astype(f32), 75)       # beyond the cache
        with pytest.raises(OgmError):
            dev.forward_all_logits(None, 0, tok_embd=emb, tokens=np.array([1, 400], np.uint32))   # id outside the vocabulary
        be.evict(emb)
    finally:
        dev.close()


@pytest.mark.parametrize("hd,group,n_kv,n_tokens,pos0", [(128, 4, 2, 200, 0), (64, 4, 2, 77, 0), (128, 1, 2, 130, 31),
                                                        (64, 5, 1, 33, 64), (128, 8, 1, 65, 7), (64, 2, 4, 300, 100)])
def test_prefill_attention_kernels_agree(be, hd, group, n_kv, n_tokens, pos0):
    """The matrix-core attention of a prefill batch (q and the probabilities as two f16 terms each,
    running softmax over tiles of 64 positions) against the decode step's kernel run per token
    (f32 multiply-adds, chunks of 128 merged afterwards): one layer, so that the cache rows do not
    depend on attention, and outputs that agree to f32 rounding.  Dropping either low-order term
    would show as 1e-4."""
    n_head = group * n_kv
    n_embd = n_head * hd
    wtype = Q4_K if n_embd % 256 == 0 else Q8_0
    outs = []
    for variant in (2, 1):   # the matrix-core kernel whatever the batch size, then the per-token one
        ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=256, n_layer=1,
                              types=(wtype, wtype, wtype, wtype), max_ctx=pos0 + n_tokens, seed=5,
                              attn_norm_scale=TAME.get(wtype, 1.0))
        be.set_tuning("attn_prefill_variant", variant)
        try:
            if pos0:
                dev.prefill(rng.standard_normal((pos0, n_embd)).astype(f32), 0)
            logits, _ = dev.prefill(rng.standard_normal((n_tokens, n_embd)).astype(f32), pos0)
            outs.append((np.asarray(logits, np.float64), np.asarray(dev.hidden(), np.float64)))
        finally:
            be.set_tuning("attn_prefill_variant", 0)
            dev.close()
    for name, a, b in (("logits", outs[0][0], outs[1][0]), ("hidden state", outs[0][1], outs[1][1])):
        err = np.abs(a - b).max() / np.abs(b).max()
        say(f"attention kernels hd {hd} group {group} {n_tokens} tokens from {pos0}: {name} differ by {err:.2e}")
        assert err <= 2e-5, f"{name}: the two attention kernels differ by {err:.3e}"


@pytest.mark.parametrize("hd,group,n_kv,n_tokens,pos0,chunks", [(128, 4, 2, 5, 700, 2), (64, 8, 1, 9, 1300, 3),
                                                                (128, 2, 2, 4, 517, 64), (128, 1, 8, 6, 1990, 0)])
def test_batch_attention_with_several_chunks_per_workgroup(be, hd, group, n_kv, n_tokens, pos0, chunks):
    """A small batch over a longer cache (a verify batch): the per-token kernel whose workgroups take several chunks
    of the cache in a row (forced: 2, 3, more than there are; the last case by the launch's own rule, 6 tokens x 16
    chunks x 8 heads) against the matrix-core kernel, as above.  Tokens of a batch that end in different chunks have
    different numbers of partial results."""
    n_head = group * n_kv
    n_embd = n_head * hd
    wtype = Q4_K if n_embd % 256 == 0 else Q8_0
    outs = []
    for variant in (2, 1):
        ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=256, n_layer=1,
                              types=(wtype, wtype, wtype, wtype), max_ctx=pos0 + n_tokens, seed=15,
                              attn_norm_scale=TAME.get(wtype, 1.0))
        be.set_tuning("attn_prefill_variant", variant)
        be.set_tuning("attn_decode_chunks", chunks)
        try:
            dev.prefill(rng.standard_normal((pos0, n_embd)).astype(f32), 0)
            be.set_tuning("attn_prefill_variant", variant)
            logits, _ = dev.prefill(rng.standard_normal((n_tokens, n_embd)).astype(f32), pos0)
            outs.append((np.asarray(logits, np.float64), np.asarray(dev.hidden(), np.float64)))
        finally:
            be.set_tuning("attn_prefill_variant", 0)
            be.set_tuning("attn_decode_chunks", 0)
            dev.close()
    for name, a, b in (("logits", outs[0][0], outs[1][0]), ("hidden state", outs[0][1], outs[1][1])):
        err = np.abs(a - b).max() / np.abs(b).max()
        say(f"batch attention, {chunks} chunks a workgroup, hd {hd} group {group} {n_tokens} tokens from {pos0}: {name} differ by {err:.2e}")
        assert err <= 2e-5, f"{name}: the two attention kernels differ by {err:.3e}"


@pytest.mark.parametrize("hd", [128, 64])
def test_prefill_attention_with_queries_beyond_f16(be, hd):
    """Per-head norms that leave q at magnitudes up to 1.5e5 (an f16 holds 65504) and k around 1e-3:
    the matrix-core kernel scales such a query row by a power of two before it splits it into f16
    terms and scales the scores back, exactly; the per-token f32 kernel needs nothing of the kind.
    They must still agree (and be finite)."""
    n_head, n_kv = 4, 2
    n_embd = n_head * hd
    wtype = Q4_K if n_embd % 256 == 0 else Q8_0
    outs = []
    for variant in (2, 1):   # the matrix-core kernel whatever the batch size, then the per-token one
        ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=256, n_layer=1,
                              types=(wtype, wtype, wtype, wtype), max_ctx=150, seed=9, pre=("q_norm", "k_norm"),
                              pre_scale={"q_norm": 4e4, "k_norm": 1e-3}, attn_norm_scale=TAME.get(wtype, 1.0))
        be.set_tuning("attn_prefill_variant", variant)
        try:
            logits, _ = dev.prefill(rng.standard_normal((150, n_embd)).astype(f32), 0)
            outs.append(np.asarray(dev.hidden(), np.float64))
        finally:
            be.set_tuning("attn_prefill_variant", 0)
            dev.close()
    assert np.isfinite(outs[0]).all() and np.isfinite(outs[1]).all()
    err = np.abs(outs[0] - outs[1]).max() / np.abs(outs[1]).max()
    say(f"large q, hd {hd}: hidden states of the two attention kernels differ by {err:.2e}")
    assert err <= 2e-5


def model_gguf(ref, arch, *, n_ctx=4096, tok_embd=None, vec_type=0, omit=(), extra_kvs=(), explicit=True,
               override_kvs=None):
    """A reference model as the bytes of a GGUF file with the tensor names and metadata keys
    LlamaModel::load_with_backend and read_model_config read (llama.rs:123-220, loader.rs:1652-1714).
    vec_type 0 stores the vectors as F32, 1 as F16."""
    from test_gguf_cpu import gguf, gstr, kv, tensor_info, u32, u64
    f32kv = lambda k, v: kv(f"{arch}.{k}", 6, np.float32(v).tobytes())
    u32kv = lambda k, v: kv(f"{arch}.{k}", 4, u32(v))
    kvs = [kv("general.architecture", 8, gstr(arch)), u32kv("embedding_length", ref.n_embd),
           u32kv("block_count", len(ref.layers)), u32kv("attention.head_count", ref.n_head),
           u32kv("context_length", n_ctx), f32kv("rope.freq_base", ref.rope_freq_base),
           f32kv("attention.layer_norm_rms_epsilon", ref.rms_eps)]
    if explicit:   # otherwise the loader's defaults must give the same model
        kvs += [u32kv("attention.head_count_kv", ref.n_head_kv), u32kv("attention.key_length", ref.head_dim),
                u32kv("rope.dimension_count", ref.rope_dim), u32kv("vocab_size", ref.n_vocab)]
    else:
        kvs.append(kv("tokenizer.ggml.tokens", 9, u32(8) + u64(ref.n_vocab) + b"".join(gstr("t%d" % i) for i in range(ref.n_vocab))))
    kvs += list(extra_kvs)
    if override_kvs:   # {key suffix: encoded key/value}: replaces that key's entry
        kvs = [k for k in kvs if not any(k.startswith(gstr(f"{arch}.{suffix}")) for suffix in override_kvs)]
        kvs += list(override_kvs.values())
    tensors = []

    def mat(name, w):
        t, raw, n_in, n_out = w
        tensors.append((name, [n_in, n_out], t, np.ascontiguousarray(raw).tobytes()))

    def vec(name, a):
        a = np.asarray(a, f32)
        tensors.append((name, [a.size], vec_type, (a if vec_type == 0 else a.astype(np.float16)).tobytes()))

    mat("token_embd.weight", tok_embd if tok_embd is not None else ref.output)
    if tok_embd is not None:
        mat("output.weight", ref.output)
    vec("output_norm.weight", ref.output_norm)
    if ref.rope_freq_factors is not None:
        vec("rope_freqs.weight", ref.rope_freq_factors)
    for i, L in enumerate(ref.layers):
        for name, field in (("attn_q", "wq"), ("attn_k", "wk"), ("attn_v", "wv"), ("attn_output", "wo"),
                            ("ffn_gate", "w_gate"), ("ffn_up", "w_up"), ("ffn_down", "w_down")):
            mat(f"blk.{i}.{name}.weight", getattr(L, field))
        for name, field in (("attn_norm.weight", "attn_norm"), ("ffn_norm.weight", "ffn_norm"), ("attn_q.bias", "q_bias"),
                            ("attn_k.bias", "k_bias"), ("attn_v.bias", "v_bias"), ("attn_q_norm.weight", "q_norm"),
                            ("attn_k_norm.weight", "k_norm")):
            if getattr(L, field) is not None:
                vec(f"blk.{i}.{name}", getattr(L, field))
    tensors = [t for t in tensors if t[0] not in omit]
    infos, blobs, pos = [], [], 0
    for name, dims, t, data in tensors:
        infos.append(tensor_info(name, dims, t, pos))
        blobs.append(data + b"\0" * ((-len(data)) % 32))
        pos += len(blobs[-1])
    return gguf(kvs, infos, data=b"".join(blobs))[0]


def f16_exact(ref):
    """Rounds every vector of the model to f16 values, so that a file storing them as F16 holds
    the same model."""
    r16 = lambda a: None if a is None else np.asarray(a, f32).astype(np.float16).astype(f32)
    ref.output_norm = r16(ref.output_norm)
    ref.rope_freq_factors = r16(ref.rope_freq_factors)
    for L in ref.layers:
        for field in ("attn_norm", "ffn_norm", "q_bias", "k_bias", "v_bias", "q_norm", "k_norm"):
            setattr(L, field, r16(getattr(L, field)))


@pytest.mark.parametrize("arch,pre,ff,vec_type,explicit,tied", [
    ("llama", (), True, 0, True, False),                                   # Llama-3.1-like: NORM pairs, rope_freqs
    ("mistral", (), False, 1, False, True),                                # defaults, tied embeddings, F16 vectors
    ("qwen2", ("q_bias", "k_bias", "v_bias"), False, 0, True, True),       # NEOX pairs, biases
    ("qwen3", ("q_norm", "k_norm"), False, 1, True, False),                # per-head norms
])
def test_a_gguf_file_decodes_like_the_model_it_holds(be, tmp_path, arch, pre, ff, vec_type, explicit, tied):
    """ogm_llama_load_gguf: hyperparameters, tensors, pairing and optional tensors as
    read_model_config and LlamaModel::load_with_backend take them from the file."""
    from orangu_amd import LlamaDecoder
    from orangu_amd.gguf import GgufFile
    n_head, n_kv, hd = (4, 4, 64) if not explicit else (8, 2, 64)   # the defaults: n_kv = n_head, head_dim = n_embd / n_head
    n_embd = 256 if not explicit else 512
    neox = arch not in ("llama", "mistral")
    factors = np.linspace(1.0, 4.0, hd // 2).astype(f32) if ff else None
    ref, dev0, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=512, n_vocab=320, n_layer=2,
                           types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=8, seed=31 + len(pre), pre=pre, neox=neox,
                           freq_factors=factors)
    dev0.close()
    if vec_type == 1:
        f16_exact(ref)
    embd = None if tied else (Q8_0, synth_weights(Q8_0, n_embd, 320, seed=77), n_embd, 320)
    path = tmp_path / f"{arch}.gguf"
    path.write_bytes(model_gguf(ref, arch, tok_embd=embd, vec_type=vec_type, explicit=explicit))
    g = GgufFile(str(path))
    dev = LlamaDecoder.from_gguf(be, g, max_ctx=8)
    try:
        c = dev.config
        assert (c.n_layer, c.n_embd, c.n_head, c.n_head_kv, c.head_dim, c.n_ff, c.n_vocab, c.rope_dim, c.rope_neox) == \
               (2, n_embd, n_head, n_kv, hd, 512, 320, hd, int(neox))
        for pos in range(3):
            step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), pos, f"{arch} file pos {pos}")
        # the embedding matrix handed back is the file's token_embd (the output matrix when tied)
        import oracle
        t, raw, _, _ = embd if embd is not None else ref.output
        want = oracle.dequantize(t, raw, 320 * n_embd).reshape(320, n_embd)[5:7]
        assert np.array_equal(be.dequant_rows(dev.tok_embd, 5, 2, in_dim=n_embd).view(np.uint32), want.view(np.uint32))
    finally:
        dev.close()
        g.close()


def test_gguf_model_loading_errors(be, tmp_path):
    """The loader's refusals (loader.rs:312-380, 1647-1681; llama.rs:186-201) arrive as a status
    and a message, not as a crash."""
    from orangu_amd import LlamaDecoder, OgmError
    from orangu_amd.gguf import GgufFile
    from test_gguf_cpu import gstr, kv, u32
    ref, dev0, rng = build(be, n_embd=256, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=320, n_layer=1,
                           types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=8, seed=41,
                           freq_factors=np.ones(32, f32))
    dev0.close()

    def load(data):
        g = GgufFile(data=data)
        try:
            LlamaDecoder.from_gguf(be, g, max_ctx=8).close()
        finally:
            g.close()

    load(model_gguf(ref, "llama"))   # the file itself is fine
    for what, data in [
        ("not a Llama-style", model_gguf(ref, "gemma")),
        ("missing tensor 'blk.0.ffn_up.weight'", model_gguf(ref, "llama", omit=("blk.0.ffn_up.weight",))),
        ("missing tensor 'output_norm.weight'", model_gguf(ref, "llama", omit=("output_norm.weight",))),
    ]:
        with pytest.raises(OgmError, match=what):
            load(data)
    ref.rope_freq_factors = np.ones(8, f32)      # fewer than rope_dim / 2 entries
    with pytest.raises(OgmError, match="rope_freqs.weight"):
        load(model_gguf(ref, "llama"))
    ref.rope_freq_factors = None
    ref.n_head = 0                               # head_count must be nonzero
    with pytest.raises(OgmError, match="nonzero"):
        load(model_gguf(ref, "llama"))
    ref.n_head = 4
    # hyperparameters that do not fit 32 bits (or whose product does not) are refused before any upload
    from test_gguf_cpu import u64
    for key, value in (("attention.head_count", 1 << 32), ("attention.head_count_kv", (1 << 32) + 2),
                       ("attention.key_length", 1 << 31), ("rope.dimension_count", 1 << 40)):
        with pytest.raises(OgmError, match="out of range"):
            load(model_gguf(ref, "llama", override_kvs={key: kv(f"llama.{key}", 10, u64(value))}))


@pytest.mark.parametrize("t,in_dim,out_dim", [
    (Q8_0, 64, 5), (Q8_0, 4096, 70),
    (Q4_K, 256, 3), (Q4_K, 1024, 130), (Q4_K, 4096, 67),
    (Q6_K, 256, 1), (Q6_K, 768, 65), (Q6_K, 4096, 129),
    (Q5_K, 256, 2), (Q5_K, 1280, 70), (Q5_K, 4096, 33),
    (Q3_K, 256, 2), (Q3_K, 1280, 70), (Q3_K, 4096, 33),
    (Q4_0, 64, 5), (Q4_0, 4096, 70), (Q5_0, 96, 66), (Q5_0, 4096, 33), (IQ4_NL, 64, 5), (IQ4_NL, 896, 130),
])
def test_dequant_rows_bits(be, t, in_dim, out_dim):
    """Rows of the device copy equal dequantize_q8_0 / _q4_k / _q6_k (quant.rs:639-787) bit for bit."""
    import oracle
    from orangu_amd import OgmError, QuantMatrix
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim + t)
    want = oracle.dequantize(t, raw, in_dim * out_dim).reshape(out_dim, in_dim)
    w = QuantMatrix(raw, t, in_dim, out_dim)
    got = be.dequant_rows(w, 0, out_dim)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    if out_dim > 2:
        got = be.dequant_rows(w, out_dim - 2, 2)
        assert np.array_equal(got.view(np.uint32), want[-2:].view(np.uint32))
    with pytest.raises(OgmError):
        be.dequant_rows(w, out_dim, 1)


@pytest.mark.parametrize("embd_t", [Q3_K, Q4_K, Q5_K, Q6_K, Q8_0, Q4_0, Q5_0, IQ4_NL])
def test_generate_matches_stepwise(be, embd_t):
    """Greedy generation on the device = the oracle's loop: embedding row of the token
    (llama.rs:609-614), decode step, last-of-equal argmax (sampling.rs:336-343)."""
    import oracle
    from orangu_amd import OgmError, QuantMatrix
    n_embd, n_vocab, max_ctx = 256, 320, 16
    kw = dict(n_embd=n_embd, n_head=4, n_kv=2, hd=64, n_ff=512, n_vocab=n_vocab, n_layer=2,
              types=(Q4_K, Q6_K, Q6_K, Q6_K), max_ctx=max_ctx, seed=11)
    ref, dev, _ = build(be, **kw)
    _, dev2, _ = build(be, **kw)
    first, steps = 17, 6
    try:
        # the first embedding seed whose greedy path is decided by more than the tolerance at every step
        for embd_seed in range(4242 + embd_t, 4242 + embd_t + 400, 50):
            embd_raw = synth_weights(embd_t, n_embd, n_vocab, seed=embd_seed)
            table = oracle.dequantize(embd_t, embd_raw, n_embd * n_vocab).reshape(n_vocab, n_embd)
            ref.reset()
            tok, want, logits, sure = first, [], None, True
            for pos in range(steps):
                logits, _ = R.decode_step(ref, table[tok], pos)
                top = np.sort(logits)[-2:]
                sure = sure and top[1] - top[0] > TOL * np.abs(logits).max()
                tok = R.argmax(logits)
                want.append(tok)
            if sure:
                break
        embd = QuantMatrix(embd_raw, embd_t, n_embd, n_vocab)
        assert sure, "no seed found: the oracle's two best logits are within the tolerance"
        got, got_logits = dev.generate(embd, first, 0, steps, want_logits=True)
        say("generated", got.tolist(), "want", want)
        assert got.tolist() == want
        close(got_logits, logits, "logits of the last generated step")
        # the same through single steps fed from the host
        tok = first
        for pos in range(steps):
            _, tok = dev2.decode(table[tok], pos)
            assert tok == want[pos]
        with pytest.raises(OgmError):
            dev.generate(embd, n_vocab, 0, 1)
        with pytest.raises(OgmError):
            dev.generate(embd, 0, max_ctx - 1, 2)
    finally:
        dev.close()
        dev2.close()


def _random_models(n, seed):
    rng = np.random.default_rng(seed)
    combos = [(Q4_K, Q6_K, Q6_K, Q6_K), (Q8_0, Q8_0, Q8_0, Q8_0), (Q5_K, Q5_K, Q6_K, Q5_K), (Q4_0, Q5_0, IQ4_NL, Q8_0)]
    out = []
    for i in range(n):
        types = combos[int(rng.integers(len(combos)))]
        hd = int(rng.choice((64, 128)))
        n_kv = int(rng.choice((1, 2, 3)))
        group = int(rng.choice((1, 2, 3, 4, 5, 8)))
        n_embd = int(rng.choice((256, 512, 768, 1280)))
        n_ff = int(rng.choice((256, 768, 1792, 2816, 11008)))
        T = int(rng.choice((1, 2, 5, 6, 9, 17, 33, 70)))
        if n_kv * group * hd % 256 != 0 and types[0] not in (Q8_0, Q4_0):   # wo's input must be whole K-quant blocks
            group = 4 if hd == 64 else 2
        out.append(pytest.param(types, hd, n_kv, group, n_embd, n_ff, T, i,
                                id=f"{i}-hd{hd}-kv{n_kv}-g{group}-e{n_embd}-ff{n_ff}-T{T}"))
    return out


@pytest.mark.parametrize("types,hd,n_kv,group,n_embd,n_ff,T,i", _random_models(28, 4242))
def test_a_seeded_walk_over_model_shapes(be, types, hd, n_kv, group, n_embd, n_ff, T, i):
    """Widths of the residual stream, of the heads together (not n_embd: Qwen3) and of the FFN drawn independently,
    FFN widths of an odd number of blocks (11008) among them; a prompt of T tokens, then two decode steps."""
    n_head = group * n_kv
    ref, dev, rng = build(be, n_embd=n_embd, n_head=n_head, n_kv=n_kv, hd=hd, n_ff=n_ff, n_vocab=320, n_layer=1,
                          types=types, max_ctx=T + 4, seed=900 + i, attn_norm_scale=TAME.get(types[0], 1.0),
                          neox=bool(i & 1), pre=("q_norm", "k_norm") if i % 3 == 0 else ())
    try:
        prefill_both(ref, dev, rng.standard_normal((T, n_embd)).astype(f32), 0, f"model {i}")
        for pos in (T, T + 1):
            step_both(ref, dev, rng.standard_normal(n_embd).astype(f32), pos, f"model {i} pos {pos}")
    finally:
        dev.close()

"""Pins the CPU restatement of the decode step's element-wise functions (oracle/llama_ref.py)
against the values the reference's own tests hold and against closed forms."""
import math

import numpy as np
import pytest

from oracle import llama_ref as R

f32 = np.float32


def test_rmsnorm_reference_case_and_closed_forms():
    # tensor.rs:1450-1466: rows [3, 4] and [0, 0], weight ones, eps 1e-5
    eps = 1e-5
    rms = math.sqrt(12.5 + eps)
    got = R.rmsnorm(np.array([3.0, 4.0], f32), np.ones(2, f32), eps)
    assert abs(got[0] - 3.0 / rms) < 1e-6 and abs(got[1] - 4.0 / rms) < 1e-6
    assert np.array_equal(R.rmsnorm(np.zeros(2, f32), np.ones(2, f32), eps), np.zeros(2, f32))
    # a constant row c: out_i = c / sqrt(c^2 + eps) * w_i
    w = np.linspace(0.5, 1.5, 64).astype(f32)
    got = R.rmsnorm(np.full(64, 2.5, f32), w, 1e-6)
    np.testing.assert_allclose(got, 2.5 / math.sqrt(6.25 + 1e-6) * w, rtol=2e-7)
    # the weight multiplies after the scale: (v * scale) * w, and a sign flip of x flips the output
    x = np.random.default_rng(1).standard_normal(256).astype(f32)
    np.testing.assert_array_equal(R.rmsnorm(-x, w.repeat(4), 1e-5), -R.rmsnorm(x, w.repeat(4), 1e-5))
    ref = x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5) * w.repeat(4)
    np.testing.assert_allclose(R.rmsnorm(x, w.repeat(4), 1e-5), ref, rtol=1e-6)


def test_rope_reference_case_and_invariants():
    # tensor.rs:1752-1769: [1..8], one head of 8, position 3, base 10000, NORM pairs
    x = np.arange(1, 9, dtype=f32)
    want = x.astype(np.float64).copy()
    for p in range(4):
        theta = 3.0 * float(f32(10000.0) ** f32(-2.0 * p / 8.0))
        a, b = want[2 * p], want[2 * p + 1]
        want[2 * p], want[2 * p + 1] = a * math.cos(theta) - b * math.sin(theta), a * math.sin(theta) + b * math.cos(theta)
    np.testing.assert_allclose(R.rope_norm(x, 1, 8, 3, 8, 10000.0), want, atol=1e-6)
    # position 0 is the identity (tensor.rs:1668); pair norms are preserved (:1676)
    y = np.random.default_rng(2).standard_normal(4 * 16).astype(f32)
    np.testing.assert_array_equal(R.rope_norm(y, 4, 16, 0, 16, 500000.0), y)
    r = R.rope_norm(y, 4, 16, 77, 16, 500000.0).reshape(-1, 2)
    np.testing.assert_allclose((r ** 2).sum(1), (y.reshape(-1, 2) ** 2).sum(1), rtol=1e-6)
    # pair 0 has frequency 1: (1, 0) at position p becomes (cos p, sin p)
    e = np.zeros(8, f32)
    e[0] = 1.0
    r = R.rope_norm(e, 1, 8, 2, 8, 10000.0)
    assert abs(r[0] - math.cos(2.0)) < 1e-6 and abs(r[1] - math.sin(2.0)) < 1e-6
    # dimensions past rope_dim are left alone; every head gets the same rotation
    r = R.rope_norm(y, 4, 16, 5, 8, 10000.0).reshape(4, 16)
    np.testing.assert_array_equal(r[:, 8:], y.reshape(4, 16)[:, 8:])
    one = R.rope_norm(y.reshape(4, 16)[2], 1, 16, 5, 8, 10000.0)
    np.testing.assert_array_equal(r[2], one)
    # rotations compose: position a then position b equals position a + b (to rounding)
    ab = R.rope_norm(R.rope_norm(y, 4, 16, 3, 16, 10000.0), 4, 16, 4, 16, 10000.0)
    np.testing.assert_allclose(ab, R.rope_norm(y, 4, 16, 7, 16, 10000.0), atol=2e-6)


def test_rope_neox_pairs_and_frequency_factors():
    # tensor.rs:1731-1749: [1..8], one head of 8, position 3, NEOX: pair p is elements p and p + 4
    x = np.arange(1, 9, dtype=f32)
    want = x.astype(np.float64).copy()
    for p in range(4):
        theta = 3.0 * float(f32(10000.0) ** f32(-2.0 * p / 8.0))
        a, b = want[p], want[p + 4]
        want[p], want[p + 4] = a * math.cos(theta) - b * math.sin(theta), a * math.sin(theta) + b * math.cos(theta)
    got = R.rope(x, 1, 8, 3, 8, 10000.0, neox=True)
    np.testing.assert_allclose(got, want, atol=1e-6)
    assert not np.array_equal(got, R.rope(x, 1, 8, 3, 8, 10000.0))        # :1771-1776: the layouts differ
    # NEOX with rope_dim < head_dim: pairs (i, i + rope_dim/2), the tail is left alone
    y = np.random.default_rng(5).standard_normal(2 * 16).astype(f32)
    r = R.rope(y, 2, 16, 9, 8, 10000.0, neox=True).reshape(2, 16)
    np.testing.assert_array_equal(r[:, 8:], y.reshape(2, 16)[:, 8:])
    np.testing.assert_allclose(r[:, :4] ** 2 + r[:, 4:8] ** 2, y.reshape(2, 16)[:, :4] ** 2 + y.reshape(2, 16)[:, 4:8] ** 2,
                               rtol=1e-5)
    # tensor.rs:1785-1822: a factor of 32 turns pair 1 of a 4-wide rotation 32 times slower, in
    # both layouts; a factor of 1 is the same bits as no factors
    for neox, a_slot in ((True, 1), (False, 2)):
        def angle(ff):
            e = np.zeros(4, f32)
            e[a_slot] = 1.0
            return float(R.rope(e, 1, 4, 1, 4, 10000.0, ff, neox)[3])
        plain, slowed = angle(None), angle(np.array([1.0, 32.0], f32))
        assert plain > 0 and slowed > 0 and abs(plain / slowed - 32.0) < 1e-2
        assert angle(np.array([1.0, 1.0], f32)) == plain
    # both layouts keep the energy of the rotated block (:1825-1841)
    z = np.array([1.0, -2.0, 3.0, 4.0, -5.0, 6.0, 7.0, -8.0], f32)
    for neox in (False, True):
        np.testing.assert_allclose((R.rope(z, 1, 8, 7, 8, 10000.0, neox=neox) ** 2).sum(), (z ** 2).sum(), rtol=1e-6)


def test_head_rmsnorm_and_biases_in_the_step():
    # per-head norm = rmsnorm of each head_dim row with one weight vector (llama.rs:770-787)
    rng = np.random.default_rng(6)
    x = rng.standard_normal(3 * 8).astype(f32)
    w = rng.uniform(0.5, 1.5, 8).astype(f32)
    got = R.head_rmsnorm(x, w, 3, 8, 1e-6).reshape(3, 8)
    for h in range(3):
        row = x.reshape(3, 8)[h].astype(np.float64)
        np.testing.assert_allclose(got[h], row / np.sqrt((row ** 2).mean() + 1e-6) * w, rtol=1e-6)
    # scaling one head leaves the others' outputs alone and (eps aside) its own too
    x2 = x.copy().reshape(3, 8)
    x2[1] *= 7.0
    got2 = R.head_rmsnorm(x2.reshape(-1), w, 3, 8, 1e-12).reshape(3, 8)
    np.testing.assert_array_equal(got2[0], R.head_rmsnorm(x, w, 3, 8, 1e-12).reshape(3, 8)[0])
    np.testing.assert_allclose(got2[1], R.head_rmsnorm(x, w, 3, 8, 1e-12).reshape(3, 8)[1], rtol=1e-5)


def test_softmax_silu_argmax():
    s = R.softmax(np.array([1.0, 2.0, 3.0], f32))           # tensor.rs:1612-1619
    assert abs(float(s.sum()) - 1.0) < 1e-6 and s[0] < s[1] < s[2]
    np.testing.assert_allclose(s, np.exp([-2.0, -1.0, 0.0]) / np.exp([-2.0, -1.0, 0.0]).sum(), rtol=1e-6)
    assert abs(float(R.silu(f32(0.0)))) < 1e-6                 # tensor.rs:1621-1625
    assert abs(float(R.silu(f32(1.0))) - 0.7310586) < 1e-6
    assert abs(float(R.silu(f32(-1.0))) + 0.26894143) < 1e-6
    assert R.argmax(np.array([1.0, 5.0, 2.0, 5.0, 0.0], f32)) == 3   # last of equal maxima
    assert R.argmax(np.array([-3.0], f32)) == 0
    # max_by over total_cmp (sampling.rs:336-343): -NaN < -inf < ... < -0 < +0 < ... < +inf < +NaN
    nan, inf = f32("nan"), f32("inf")
    neg_nan = np.array([0xFFC00000], np.uint32).view(f32)[0]
    assert R.argmax(np.array([1.0, nan, 7.0], f32)) == 1
    assert R.argmax(np.array([-0.0, 0.0, -0.0], f32)) == 1
    assert R.argmax(np.array([0.0, -0.0], f32)) == 0
    assert R.argmax(np.array([neg_nan, -inf, neg_nan], f32)) == 1
    assert R.argmax(np.array([neg_nan, neg_nan], f32)) == 1
    assert R.argmax(np.array([inf, 3.0, inf], f32)) == 2


def test_cache_rows_saturate_at_the_f16_range():
    row = np.array([1.0, 65504.0, 65519.0, 65520.0, 1e9, -1e9, np.inf, -np.inf, np.nan], f32)
    got = R.to_cache(row, np.float16)
    assert got.dtype == np.float16
    np.testing.assert_array_equal(got[:8].astype(f32), [1.0, 65504.0, 65504.0, 65504.0, 65504.0, -65504.0, 65504.0, -65504.0])
    assert np.isnan(got[8])
    np.testing.assert_array_equal(R.to_cache(row, f32)[:6], row[:6])   # the reference's f32 cache keeps everything


def test_attention_closed_forms_and_head_mapping():
    rng = np.random.default_rng(3)
    n_head, n_kv, hd = 4, 2, 8
    q = rng.standard_normal(n_head * hd).astype(f32)
    # a single cached position: out_h = v[kv head of h]
    k1, v1 = rng.standard_normal((1, n_kv * hd)).astype(f32), rng.standard_normal((1, n_kv * hd)).astype(f32)
    out = R.attention(q, k1, v1, n_head, n_kv, hd).reshape(n_head, hd)
    for h in range(n_head):
        np.testing.assert_allclose(out[h], v1.reshape(n_kv, hd)[h // 2], rtol=1e-6)
    # equal scores (all keys the same): the mean of the values
    k = np.tile(k1, (5, 1))
    v = rng.standard_normal((5, n_kv * hd)).astype(f32)
    out = R.attention(q, k, v, n_head, n_kv, hd).reshape(n_head, hd)
    for h in range(n_head):
        np.testing.assert_allclose(out[h], v.reshape(5, n_kv, hd)[:, h // 2].mean(0), rtol=1e-5, atol=1e-6)
    # brute force in float64 with the explicit head mapping
    k = rng.standard_normal((9, n_kv * hd)).astype(f32)
    v = rng.standard_normal((9, n_kv * hd)).astype(f32)
    out = R.attention(q, k, v, n_head, n_kv, hd).reshape(n_head, hd)
    for h in range(n_head):
        kh, vh = k.reshape(9, n_kv, hd)[:, h // 2].astype(np.float64), v.reshape(9, n_kv, hd)[:, h // 2].astype(np.float64)
        sc = kh @ q.reshape(n_head, hd)[h].astype(np.float64) / math.sqrt(hd)
        w = np.exp(sc - sc.max())
        w /= w.sum()
        np.testing.assert_allclose(out[h], w @ vh, rtol=1e-5, atol=1e-6)
    # one overwhelming key: its value wins
    k[4] = 50.0 * np.tile(q.reshape(n_head, hd)[:: 2].reshape(-1) / np.linalg.norm(q), 1)[: n_kv * hd]
    out = R.attention(q, k, v, n_head, n_kv, hd).reshape(n_head, hd)
    np.testing.assert_allclose(out[0], v.reshape(9, n_kv, hd)[4, 0], atol=1e-3)


def test_decode_step_wiring_on_a_tiny_model():
    """Two layers by hand: the residual stream, the cache growth and the f16 cache rounding."""
    from helpers import Q4_K, Q6_K, synth_weights
    rng = np.random.default_rng(4)
    n_embd, n_head, n_kv, hd, n_ff, n_vocab = 256, 4, 2, 64, 512, 320
    mk = lambda t, i, o, s: (t, synth_weights(t, i, o, seed=s), i, o)
    layers = [R.Layer(mk(Q4_K, n_embd, n_head * hd, 1 + 10 * l), mk(Q4_K, n_embd, n_kv * hd, 2 + 10 * l),
                      mk(Q6_K, n_embd, n_kv * hd, 3 + 10 * l), mk(Q4_K, n_head * hd, n_embd, 4 + 10 * l),
                      mk(Q4_K, n_embd, n_ff, 5 + 10 * l), mk(Q4_K, n_embd, n_ff, 6 + 10 * l),
                      mk(Q6_K, n_ff, n_embd, 7 + 10 * l),
                      (1 + 0.1 * rng.standard_normal(n_embd)).astype(f32),
                      (1 + 0.1 * rng.standard_normal(n_embd)).astype(f32)) for l in range(2)]
    m = R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd, 1e-5, 10000.0, layers,
                np.ones(n_embd, f32), mk(Q6_K, n_embd, n_vocab, 99))
    x0, x1 = rng.standard_normal(n_embd).astype(f32), rng.standard_normal(n_embd).astype(f32)
    lg0, h0 = R.decode_step(m, x0, 0)
    lg1, h1 = R.decode_step(m, x1, 1)
    assert lg0.shape == (n_vocab,) and h1.shape == (n_embd,) and np.isfinite(lg1).all()
    assert [len(c) for c in m.k_cache] == [2, 2] and m.k_cache[0][0].dtype == np.float16
    # at position 0 attention returns the (f16-rounded) value row itself: rebuild layer 0 by hand
    L = layers[0]
    normed = R.rmsnorm(x0, L.attn_norm, 1e-5)
    v = R._mm(L.wv, normed).astype(np.float16).astype(f32)
    attn = np.repeat(v.reshape(n_kv, hd), n_head // n_kv, axis=0).reshape(-1)
    x = x0 + R._mm(L.wo, attn)
    n2 = R.rmsnorm(x, L.ffn_norm, 1e-5)
    x = x + R._mm(L.w_down, R.silu(R._mm(L.w_gate, n2)) * R._mm(L.w_up, n2))
    m1 = R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd, 1e-5, 10000.0, layers[:1],
                 np.ones(n_embd, f32), m.output)
    _, h = R.decode_step(m1, x0, 0)
    np.testing.assert_allclose(h, x, rtol=1e-5, atol=1e-6)
    # a decode out of order is refused
    with pytest.raises(AssertionError):
        R.decode_step(m, x0, 5)


def test_first_position_sees_only_v_and_its_bias():
    """With one cached position the softmax weight is 1 whatever q and k are: the logits at
    position 0 do not move with the q / k biases, the per-head norms, the pairing or the frequency
    factors, and do move with the v bias; at position 1 the q / k side matters."""
    from helpers import Q4_K, Q6_K, synth_weights
    import dataclasses
    rng = np.random.default_rng(8)
    n_embd, n_head, n_kv, hd, n_ff, n_vocab = 256, 4, 2, 64, 256, 64
    mk = lambda t, i, o, s: (t, synth_weights(t, i, o, seed=s), i, o)
    base = R.Layer(mk(Q4_K, n_embd, n_head * hd, 1), mk(Q4_K, n_embd, n_kv * hd, 2), mk(Q6_K, n_embd, n_kv * hd, 3),
                   mk(Q4_K, n_head * hd, n_embd, 4), mk(Q4_K, n_embd, n_ff, 5), mk(Q4_K, n_embd, n_ff, 6),
                   mk(Q6_K, n_ff, n_embd, 7), np.ones(n_embd, f32), np.ones(n_embd, f32))
    qk = dict(q_bias=rng.standard_normal(n_head * hd).astype(f32), k_bias=rng.standard_normal(n_kv * hd).astype(f32),
              q_norm=rng.uniform(0.5, 2, hd).astype(f32), k_norm=rng.uniform(0.5, 2, hd).astype(f32))

    def run(layer, **kw):
        m = R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd, 1e-5, 10000.0, [layer], np.ones(n_embd, f32),
                    mk(Q6_K, n_embd, n_vocab, 9), **kw)
        x0, x1 = np.random.default_rng(9).standard_normal((2, n_embd)).astype(f32)
        return R.decode_step(m, x0, 0)[0], R.decode_step(m, x1, 1)[0]

    plain0, plain1 = run(base)
    other0, other1 = run(dataclasses.replace(base, **qk), rope_neox=True,
                         rope_freq_factors=np.linspace(1, 8, hd // 2).astype(f32))
    np.testing.assert_array_equal(other0, plain0)
    assert not np.array_equal(other1, plain1)
    vb0, _ = run(dataclasses.replace(base, v_bias=np.full(n_kv * hd, 0.5, f32)))
    assert not np.array_equal(vb0, plain0)


def test_prefill_of_several_tokens_matches_decoding_them_one_by_one():
    """forward over T rows at once (GEMM float order, llama.rs:594-932 at n_tokens > 1) against T
    single-token steps (GEMV order): the same cache rows and last logits up to f32 rounding, also
    when the batch continues a cache that already holds positions; causality: the rows of the
    earlier tokens do not move when later tokens join the batch."""
    from helpers import Q4_K, Q6_K, synth_weights
    rng = np.random.default_rng(11)
    n_embd, n_head, n_kv, hd, n_ff, n_vocab = 256, 4, 2, 64, 256, 64
    mk = lambda t, i, o, s: (t, synth_weights(t, i, o, seed=s), i, o)
    layers = [R.Layer(mk(Q4_K, n_embd, n_head * hd, 1 + 10 * l), mk(Q4_K, n_embd, n_kv * hd, 2 + 10 * l),
                      mk(Q6_K, n_embd, n_kv * hd, 3 + 10 * l), mk(Q4_K, n_head * hd, n_embd, 4 + 10 * l),
                      mk(Q4_K, n_embd, n_ff, 5 + 10 * l), mk(Q4_K, n_embd, n_ff, 6 + 10 * l),
                      mk(Q6_K, n_ff, n_embd, 7 + 10 * l), np.ones(n_embd, f32), np.ones(n_embd, f32),
                      q_bias=rng.standard_normal(n_head * hd).astype(f32)) for l in range(2)]
    new = lambda: R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd, 1e-5, 10000.0, layers, np.ones(n_embd, f32),
                          mk(Q6_K, n_embd, n_vocab, 99), rope_neox=True, kv_dtype=np.float32)
    X = rng.standard_normal((7, n_embd)).astype(f32)
    one = new()
    for t in range(7):
        lg_one, h_one = R.decode_step(one, X[t], t)
    batch = new()
    lg_b, h_b = R.forward(batch, X, 0)
    split = new()
    R.forward(split, X[:3], 0)
    lg_s, h_s = R.forward(split, X[3:], 3)
    for other, lg, h in ((batch, lg_b, h_b), (split, lg_s, h_s)):
        np.testing.assert_allclose(h, h_one, rtol=0, atol=2e-5 * np.abs(h_one).max())
        np.testing.assert_allclose(lg, lg_one, rtol=0, atol=2e-5 * np.abs(lg_one).max())
        for l in range(2):
            a, b = np.stack(other.k_cache[l]), np.stack(one.k_cache[l])
            np.testing.assert_allclose(a, b, rtol=0, atol=2e-5 * np.abs(b).max())
            a, b = np.stack(other.v_cache[l]), np.stack(one.v_cache[l])
            np.testing.assert_allclose(a, b, rtol=0, atol=2e-5 * np.abs(b).max())
    short = new()
    R.forward(short, X[:4], 0)
    for l in range(2):   # bit for bit: rows of a GEMM do not depend on the other rows of the batch
        np.testing.assert_array_equal(np.stack(short.k_cache[l]), np.stack(batch.k_cache[l])[:4])
        np.testing.assert_array_equal(np.stack(short.v_cache[l]), np.stack(batch.v_cache[l])[:4])


def test_hidden_states_are_the_normed_final_rows_of_every_prefix():
    """forward_hidden_states (llama.rs:1034-1045): row t is the output norm of the hidden state the last
    token of the prefix 0 .. t ends with -- causality makes it independent of the tokens after it (bit for
    bit: a GEMM row does not depend on the other rows) -- and of single-token steps up to f32 rounding;
    the call starts from an empty cache of its own whatever the model held before."""
    from helpers import Q4_K, Q6_K, synth_weights
    rng = np.random.default_rng(13)
    n_embd, n_head, n_kv, hd, n_ff, n_vocab = 256, 4, 2, 64, 256, 64
    mk = lambda t, i, o, s: (t, synth_weights(t, i, o, seed=s), i, o)
    layers = [R.Layer(mk(Q4_K, n_embd, n_head * hd, 1 + 10 * l), mk(Q4_K, n_embd, n_kv * hd, 2 + 10 * l),
                      mk(Q6_K, n_embd, n_kv * hd, 3 + 10 * l), mk(Q4_K, n_head * hd, n_embd, 4 + 10 * l),
                      mk(Q4_K, n_embd, n_ff, 5 + 10 * l), mk(Q4_K, n_embd, n_ff, 6 + 10 * l),
                      mk(Q6_K, n_ff, n_embd, 7 + 10 * l), np.ones(n_embd, f32), np.ones(n_embd, f32)) for l in range(2)]
    out_norm = rng.uniform(0.5, 2.0, n_embd).astype(f32)
    new = lambda: R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd, 1e-5, 10000.0, layers, out_norm,
                          mk(Q6_K, n_embd, n_vocab, 99), kv_dtype=np.float32)
    X = rng.standard_normal((6, n_embd)).astype(f32)
    m = new()
    R.forward(m, X[:2], 0)                      # a cache the call must not continue
    H = R.hidden_states(m, X)
    assert H.shape == (6, n_embd) and H.dtype == f32 and [len(c) for c in m.k_cache] == [6, 6]
    for t in (1, 3, 5):                         # prefixes of several tokens: the same GEMM kernels, the same bits
        _, h_last = R.forward(new(), X[:t + 1], 0)
        np.testing.assert_array_equal(H[t], R.rmsnorm(h_last, out_norm, 1e-5))
    one = new()
    for t in range(6):
        _, h = R.decode_step(one, X[t], t)
        want = R.rmsnorm(h, out_norm, 1e-5)
        np.testing.assert_allclose(H[t], want, rtol=0, atol=2e-5 * np.abs(want).max())
    # the norm weight enters once per element: halving one weight halves that column and no other
    out_norm2 = out_norm.copy()
    out_norm2[7] *= 0.5
    m2 = R.Model(n_embd, n_head, n_kv, hd, n_ff, n_vocab, hd, 1e-5, 10000.0, layers, out_norm2,
                 mk(Q6_K, n_embd, n_vocab, 99), kv_dtype=np.float32)
    H2 = R.hidden_states(m2, X)
    np.testing.assert_array_equal(H2[:, 7], H[:, 7] * f32(0.5))
    np.testing.assert_array_equal(np.delete(H2, 7, axis=1), np.delete(H, 7, axis=1))

"""Pins the oracle's fused GEMV / GEMM kernels and CpuBackend dispatch against the reference's own
tests (engine/vecdot.rs:3408-4812, engine/backend/cpu.rs:509-651) and against independent numpy
arithmetic.  CPU only."""
import numpy as np
import pytest

import oracle
from helpers import (BLOCK, FLAT32, IQ4_NL, Q3_K, Q4_0, Q4_K, Q5_0, Q5_K, Q6_K, Q8_0, NextByte, activations, cpu_rs_weights, fixture_row,
                     k_fixture, row_bytes)


# ---------------------------------------------------------------- integer dots

def test_dot16_known_answers():
    """vecdot.rs:577-594: the reference's own self-check vectors.  Expected values by hand:
    16, -16, sum of the third vector, and the written-out fourth product sum."""
    one = np.ones(16, np.int8)
    c3 = np.array([127, -128, 127, -128, 1, -1, 0, 64, -64, 32, -32, 16, -16, 8, -8, 2], np.int8)
    w4 = np.array([3, -5, 7, -11, 13, -17, 19, -23, 29, -31, 37, -41, 43, -47, 53, -59], np.int8)
    x4 = np.array([2, 4, -6, 8, -10, 12, 14, -16, 18, -20, 22, 24, -26, 28, 30, -32], np.int8)
    want4 = sum(int(a) * int(b) for a, b in zip(w4, x4))
    for fn in (oracle.dot16_scalar, oracle.dot16):
        assert fn(one, one) == 16
        assert fn(-one, one) == -16
        assert fn(c3, one) == int(c3.astype(int).sum()) == 0
        assert fn(w4, x4) == want4
    assert want4 == 6 - 20 - 42 - 88 - 130 - 204 + 266 + 368 + 522 + 620 + 814 - 984 - 1118 - 1316 + 1590 + 1888


def test_dot32_and_dot16_every_isa_equals_brute_force():
    rng = np.random.default_rng(1)
    for _ in range(200):
        w = rng.integers(-128, 128, 32, dtype=np.int8)
        x = rng.integers(-127, 128, 32, dtype=np.int8)
        want = int((w.astype(np.int64) * x.astype(np.int64)).sum())
        want16 = int((w[:16].astype(np.int64) * x[:16].astype(np.int64)).sum())
        for scalar in (True, False):
            oracle.force_scalar(scalar)
            assert oracle.dot32(w, x) == want
            assert oracle.dot16(w, x) == want16
        oracle.force_scalar(False)
    assert oracle.dot16_scalar(w, x) == want16


# ---------------------------------------------------------------- numpy restatement of the integer stage

def np_unpack(ggml_type, row, in_dim):
    """Independent numpy decode of a row into (q int [n], scale-per-element int [n],
    min-per-element int [n], d f32 [n_blocks], dmin f32 [n_blocks]) from ggml's published layouts."""
    bb, be = BLOCK[ggml_type]
    blocks = row.reshape(-1, bb)
    nb = blocks.shape[0]
    if ggml_type == Q8_0:
        d = blocks[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)
        q = blocks[:, 2:].copy().view(np.int8).astype(np.int64).reshape(-1)
        return q, None, None, d, None
    if ggml_type in (Q4_0, Q5_0, IQ4_NL):   # d | [qh u32] | qs[16]: low nibbles, then high nibbles
        d = blocks[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)
        qs = blocks[:, bb - 16:].astype(np.int64)
        nib = np.concatenate([qs & 15, qs >> 4], axis=1)
        if ggml_type == IQ4_NL:
            q = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.int64)[nib]
        elif ggml_type == Q4_0:
            q = nib - 8
        else:
            q = nib + 16 * np.unpackbits(blocks[:, 2:6].copy(), axis=1, bitorder="little").astype(np.int64) - 16
        return q.reshape(-1), None, None, d, None
    if ggml_type == Q4_K:
        d = blocks[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)
        dmin = blocks[:, 2:4].copy().view(np.float16).astype(np.float32).reshape(-1)
        b = blocks[:, 4:16].astype(np.int64)
        sc = np.empty((nb, 8), np.int64)
        mn = np.empty((nb, 8), np.int64)
        sc[:, :4] = b[:, 0:4] & 63
        mn[:, :4] = b[:, 4:8] & 63
        sc[:, 4:] = (b[:, 8:12] & 15) | ((b[:, 0:4] >> 6) << 4)
        mn[:, 4:] = (b[:, 8:12] >> 4) | ((b[:, 4:8] >> 6) << 4)
        qs = blocks[:, 16:].astype(np.int64).reshape(nb, 4, 32)
        q = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1)  # [nb][g][half][32]
        return q, np.repeat(sc, 32, axis=1).reshape(-1), np.repeat(mn, 32, axis=1).reshape(-1), d, dmin
    if ggml_type == Q5_K:   # Q4_K with qh[32] between the scales and qs; bit j of qh[l]: sub-block j
        q4, sce, mne, d, dmin = np_unpack(Q4_K, np.concatenate([blocks[:, :16], blocks[:, 48:]], axis=1).reshape(-1),
                                          in_dim)
        qh = blocks[:, 16:48].astype(np.int64)                                        # [nb][32]
        hi = ((qh[:, None, :] >> np.arange(8)[None, :, None]) & 1) * 16              # [nb][8][32]
        return q4 + hi.reshape(-1), sce, mne, d, dmin
    if ggml_type == Q3_K:   # hmask[32] | qs[64] | scales[12] | d; run p: qs[32 (p/4) + j] >> 2 (p%4), hmask bit p
        hm = blocks[:, 0:32].astype(np.int64)
        qs = blocks[:, 32:96].astype(np.int64).reshape(nb, 2, 32)
        pk = blocks[:, 96:108].astype(np.int64)
        d = blocks[:, 108:110].copy().view(np.float16).astype(np.float32).reshape(-1)
        q = np.empty((nb, 8, 32), np.int64)
        for p in range(8):
            q[:, p, :] = ((qs[:, p // 4, :] >> (2 * (p % 4))) & 3) - np.where((hm >> p) & 1, 0, 4)
        sc = np.empty((nb, 16), np.int64)
        for i in range(16):
            low = pk[:, i] & 15 if i < 8 else pk[:, i - 8] >> 4
            sc[:, i] = (low | (((pk[:, 8 + i % 4] >> (2 * (i // 4))) & 3) << 4)) - 32
        return q.reshape(-1), np.repeat(sc, 16, axis=1).reshape(-1), None, d, None
    ql = blocks[:, 0:128].astype(np.int64).reshape(nb, 2, 2, 32)  # [h][r&1][l]
    qh = blocks[:, 128:192].astype(np.int64).reshape(nb, 2, 32)
    sc = blocks[:, 192:208].copy().view(np.int8).astype(np.int64)
    d = blocks[:, 208:210].copy().view(np.float16).astype(np.float32).reshape(-1)
    q = np.empty((nb, 2, 4, 32), np.int64)
    for r in range(4):
        nib = ql[:, :, r & 1, :] & 15 if r < 2 else ql[:, :, r & 1, :] >> 4
        q[:, :, r, :] = (nib | (((qh >> (2 * r)) & 3) << 4)) - 32
    return q.reshape(-1), np.repeat(sc, 16, axis=1).reshape(-1), None, d, None


def np_block_sums(ggml_type, row, in_dim, xq):
    q, sce, mne, d, dmin = np_unpack(ggml_type, row, in_dim)
    xq = xq.astype(np.int64)
    if ggml_type in FLAT32:
        return (q * xq).reshape(-1, 32).sum(axis=1), None
    isum = (q * sce * xq).reshape(-1, 256).sum(axis=1)
    imin = (mne * xq).reshape(-1, 256).sum(axis=1) if mne is not None else None
    return isum, imin


@pytest.mark.parametrize("ggml_type", [Q3_K, Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("in_dim", [256, 2048])
def test_k_row_integer_sums_equal_numpy_int64(ggml_type, in_dim):
    """Per-super-block isum / imin (vecdot.rs:3152-3178, 3215-3241) against int64 numpy over an
    independently decoded row."""
    row = fixture_row(ggml_type, in_dim, 7)
    act = oracle.quantize_act_k_row(activations(in_dim))
    _, isum, imin = oracle.dot_k_row(ggml_type, row, act, want_sums=True)
    wi, wm = np_block_sums(ggml_type, row, in_dim, act[0])
    assert np.array_equal(isum, wi)
    if ggml_type in (Q4_K, Q5_K):
        assert np.array_equal(imin, wm)


def test_k_row_float_combine_is_left_to_right_f32():
    """total += act.d[s] * (d*isum - dmin*imin) (Q4_K) / act.d[s]*d*isum (Q6_K), one f32
    accumulator, each op rounded (vecdot.rs:3175, 3238), rebuilt from numpy int sums."""
    f = np.float32
    for ggml_type in (Q4_K, Q6_K):
        in_dim = 2048
        row = fixture_row(ggml_type, in_dim, 99)
        act = oracle.quantize_act_k_row(activations(in_dim))
        got = oracle.dot_k_row(ggml_type, row, act)
        isum, imin = np_block_sums(ggml_type, row, in_dim, act[0])
        _, _, _, d, dmin = np_unpack(ggml_type, row, in_dim)
        total = f(0)
        for s in range(in_dim // 256):
            if ggml_type == Q4_K:
                total = f(total + f(act[1][s] * f(f(d[s] * f(isum[s])) - f(dmin[s] * f(imin[s])))))
            else:
                total = f(total + f(f(act[1][s] * d[s]) * f(isum[s])))
        assert got.view(np.uint32) == total.view(np.uint32)


def test_q8_0_row_is_left_to_right_f32():
    """vecdot.rs:2829-2838: total += (dw * act.d[b]) * (f32)isum."""
    f = np.float32
    in_dim = 896
    row = fixture_row(Q8_0, in_dim, 1)
    act = oracle.quantize_act(activations(in_dim))
    got = oracle.dot_row(Q8_0, row, act)
    isum, _ = np_block_sums(Q8_0, row, in_dim, act[0])
    _, _, _, d, _ = np_unpack(Q8_0, row, in_dim)
    total = f(0)
    for b in range(in_dim // 32):
        total = f(total + f(f(d[b] * act[1][b]) * f(isum[b])))
    assert got.view(np.uint32) == total.view(np.uint32)


# ---------------------------------------------------------------- the reference's budget tests

def _reference(ggml_type, row, in_dim, x):
    w = oracle.dequantize(ggml_type, row, in_dim)
    prod = (w * x).astype(np.float32)
    ref = np.float32(0)
    for p in prod:  # f32 left-to-right `.sum()`
        ref = np.float32(ref + p)
    return ref, np.abs(prod.astype(np.float64)).sum()


CHECK_CASES = [(Q8_0, 896), (Q8_0, 4864), (Q4_K, 256), (Q4_K, 4864 // 256 * 256), (Q6_K, 256),
               (Q6_K, 4864 // 256 * 256)]


@pytest.mark.parametrize("ggml_type,in_dim", [(Q8_0, 896), (Q8_0, 4864), (Q4_K, 256), (Q4_K, 4864),
                                              (Q6_K, 256), (Q6_K, 4864), (Q5_0, 896), (Q5_0, 4864),
                                              (Q4_0, 32), (Q4_0, 896), (Q4_0, 4864), (IQ4_NL, 896),
                                              (IQ4_NL, 4864)])
@pytest.mark.parametrize("seed", [1, 7, 99])
def test_fused_dot_row_matches_dequantize_reference(ggml_type, in_dim, seed):
    """vecdot.rs:3436-3526 `check` via dot_row (per-32 activations): |got - ref| <= 0.01 * sum|w x|.
    4864 = 19 * 256, so it is a whole number of super-blocks for the K-quants too."""
    row = fixture_row(ggml_type, in_dim, seed)
    x = activations(in_dim)
    ref, mag = _reference(ggml_type, row, in_dim, x)
    act = oracle.quantize_act(x)
    got = oracle.dot_row(ggml_type, row, act)
    assert abs(float(got) - float(ref)) <= 0.01 * max(mag, 1e-6)


@pytest.mark.parametrize("ggml_type", [Q3_K, Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("in_dim", [256, 2048, 3072, 5632])
@pytest.mark.parametrize("seed", [1, 7, 99])
def test_k_row_decode_matches_dequantize_reference(ggml_type, in_dim, seed):
    """vecdot.rs:4011-4040 (and :4127-4133 for Q5_K): budget 0.02 * sum|w x| for the per-256 decode."""
    row = fixture_row(ggml_type, in_dim, seed)
    x = activations(in_dim)
    ref, mag = _reference(ggml_type, row, in_dim, x)
    assert oracle.supports_k_row(ggml_type, in_dim)
    got = oracle.dot_k_row(ggml_type, row, oracle.quantize_act_k_row(x))
    assert abs(float(got) - float(ref)) <= 0.02 * max(mag, 1e-6)


def test_integer_accumulators_stay_inside_i32_by_construction():
    """vecdot.rs:4094-4116 / 3068-3082: worst-case per-super-block magnitudes."""
    assert 63 * 15 * 127 * 256 < 2**31 // 8  # Q4_K isum
    assert 63 * 127 * 256 < 2**31 // 8  # Q4_K imin
    assert 127 * 32 * 127 * 256 < 2**31 // 8  # Q6_K isum (|sc|<=128 checked separately)
    assert 128 * 32 * 127 * 256 < 2**31


@pytest.mark.parametrize("ggml_type", [Q3_K, Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("in_dim", [256, 2048, 8192])
def test_k_gemm_matches_dequantize_reference(ggml_type, in_dim):
    """vecdot.rs:4479-4513: 5 rows x 7 tokens, seed 4242, budget 0.01 * sum|w x|."""
    out_dim, n_tokens = 5, 7
    raw, x = k_fixture(ggml_type, in_dim, out_dim, n_tokens, 4242)
    got = oracle.k_gemm_t(ggml_type, raw, in_dim, out_dim, x, n_tokens)
    rb = row_bytes(ggml_type, in_dim)
    for o in range(out_dim):
        w = oracle.dequantize(ggml_type, raw[o * rb:(o + 1) * rb], in_dim).astype(np.float64)
        for t in range(n_tokens):
            xs = x[t * in_dim:(t + 1) * in_dim].astype(np.float64)
            ref, mag = (w * xs).sum(), np.abs(w * xs).sum()
            assert abs(got[o, t] - ref) <= 0.01 * max(mag, 1e-6) + 1e-6 * mag


@pytest.mark.parametrize("ggml_type", [Q3_K, Q4_K, Q5_K, Q6_K])
def test_k_gemm_result_is_independent_of_the_batch_size(ggml_type):
    """vecdot.rs:4522-4549: exact equality."""
    in_dim, out_dim = 512, 4
    raw, x = k_fixture(ggml_type, in_dim, out_dim, 8, 77)
    full = oracle.k_gemm_t(ggml_type, raw, in_dim, out_dim, x, 8)
    for n in (2, 3, 5, 7):
        part = oracle.k_gemm_t(ggml_type, raw, in_dim, out_dim, x[: n * in_dim], n)
        assert np.array_equal(part.view(np.uint32), full[:, :n].view(np.uint32))


@pytest.mark.parametrize("ggml_type", [Q3_K, Q4_K, Q5_K, Q6_K])
def test_k_gemm_float_order_rebuilt_from_integer_sums(ggml_type):
    """gemm_k_q4_k: acc -= (ad*dmin)*imin over all super-blocks first, then acc += ad*(d*isum)
    (vecdot.rs:2229-2303); gemm_k_q6_k: acc += ad*(d*isum) (vecdot.rs:2386-2391).  Rebuilt in
    numpy f32 from independently computed integer sums: pins the order and the parenthesisation,
    which differ from the GEMV's."""
    f = np.float32
    in_dim, out_dim, n_tokens = 1024, 3, 5
    raw, x = k_fixture(ggml_type, in_dim, out_dim, n_tokens, 31)
    got = oracle.k_gemm_t(ggml_type, raw, in_dim, out_dim, x, n_tokens)
    rb = row_bytes(ggml_type, in_dim)
    for o in range(out_dim):
        row = raw[o * rb:(o + 1) * rb]
        _, _, _, d, dmin = np_unpack(ggml_type, row, in_dim)
        for t in range(n_tokens):
            xq, ad, _ = oracle.quantize_act_k_row(x[t * in_dim:(t + 1) * in_dim])
            isum, imin = np_block_sums(ggml_type, row, in_dim, xq)
            acc = f(0)
            if ggml_type in (Q4_K, Q5_K):
                for s in range(in_dim // 256):
                    acc = f(acc - f(f(ad[s] * dmin[s]) * f(imin[s])))
            for s in range(in_dim // 256):
                acc = f(acc + f(ad[s] * f(d[s] * f(isum[s]))))
            assert got[o, t].view(np.uint32) == acc.view(np.uint32), (o, t)


# ---------------------------------------------------------------- CpuBackend dispatch

@pytest.mark.parametrize("ggml_type", [Q8_0, Q4_K])
def test_decode_batch_is_bit_identical_to_deciding_each_token_alone(ggml_type):
    """backend/cpu.rs:623-650."""
    in_dim = 128 if ggml_type == Q8_0 else 512
    out_dim, n_tokens = 7, 5
    nb = NextByte(0x0051AB1E5EED)
    raw = cpu_rs_weights(ggml_type, in_dim, out_dim, nb)
    x = np.array([np.float32(nb()) / np.float32(255.0) * np.float32(2.0) - np.float32(1.0)
                  for _ in range(n_tokens * in_dim)], np.float32)
    batched = oracle.matmul_decode(ggml_type, raw, in_dim, out_dim, x, n_tokens)
    for t in range(n_tokens):
        alone = oracle.matmul(ggml_type, raw, in_dim, out_dim, x[t * in_dim:(t + 1) * in_dim], 1)
        assert np.array_equal(alone[0].view(np.uint32), batched[t].view(np.uint32))


@pytest.mark.parametrize("ggml_type", [Q8_0, Q4_K])
def test_matmul_dispatch_shapes_and_kernels(ggml_type):
    """backend/cpu.rs:544-582 shapes (in = 3 blocks, out = 11 odd, T in 1,2,5,77,3,1).  matmul at
    T > 1 takes the GEMM kernels: K-quants follow the two-pass GEMM order, Q8_0's flat GEMM equals
    the GEMV per token bit for bit (vecdot.rs:2594-2597)."""
    in_dim = BLOCK[ggml_type][1] * 3
    out_dim = 11
    raw = cpu_rs_weights(ggml_type, in_dim, out_dim, NextByte(0x9E3779B97F4A7C15))
    for n_tokens in (1, 2, 5, 77, 3, 1):
        i = np.arange(n_tokens * in_dim)
        x = ((i % 29).astype(np.float32) - np.float32(14.0)) * np.float32(0.037)
        y = oracle.matmul(ggml_type, raw, in_dim, out_dim, x, n_tokens)
        assert y.shape == (n_tokens, out_dim)
        yd = oracle.matmul_decode(ggml_type, raw, in_dim, out_dim, x, n_tokens)
        if ggml_type == Q8_0 or n_tokens == 1:
            assert np.array_equal(y.view(np.uint32), yd.view(np.uint32))
        else:
            yt = oracle.k_gemm_t(ggml_type, raw, in_dim, out_dim, x, n_tokens)
            assert np.array_equal(y.view(np.uint32), yt.T.view(np.uint32))
            assert np.allclose(y, yd, rtol=1e-4, atol=1e-3)


def test_threaded_matmul_equals_single_thread():
    for ggml_type in (Q8_0, Q4_K, Q6_K):
        in_dim, out_dim = 512, 37
        raw, x = k_fixture(ggml_type, in_dim, out_dim, 6, 5) if ggml_type != Q8_0 else (
            fixture_row(Q8_0, in_dim * out_dim, 5), activations(in_dim * 6))
        for T in (1, 6):
            a = oracle.matmul(ggml_type, raw, in_dim, out_dim, x[: T * in_dim], T, threads=1)
            b = oracle.matmul(ggml_type, raw, in_dim, out_dim, x[: T * in_dim], T, threads=0)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_scalar_and_avx2_builds_agree_bitwise():
    in_dim, out_dim, T = 1024, 9, 5
    for ggml_type in (Q8_0, Q4_K, Q6_K):
        raw = fixture_row(ggml_type, in_dim * out_dim, 3)
        x = activations(in_dim * T)
        oracle.force_scalar(True)
        a = oracle.matmul(ggml_type, raw, in_dim, out_dim, x, T)
        ad = oracle.matmul_decode(ggml_type, raw, in_dim, out_dim, x, T)
        oracle.force_scalar(False)
        b = oracle.matmul(ggml_type, raw, in_dim, out_dim, x, T)
        bd = oracle.matmul_decode(ggml_type, raw, in_dim, out_dim, x, T)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert np.array_equal(ad.view(np.uint32), bd.view(np.uint32))


def test_supports_predicates():
    """vecdot.rs:274-283, 1821-1826, 3083-3093, 2456-2461 for the three types."""
    assert oracle.supports(Q8_0, 96) and not oracle.supports(Q8_0, 100)
    assert oracle.supports(Q4_K, 512) and not oracle.supports(Q4_K, 896)
    for t in (Q5_0, Q4_0, IQ4_NL):   # vecdot.rs:4248-4262, 2456-2461
        assert oracle.supports(t, 896) and not oracle.supports(t, 24) and oracle.supports_flat(t, 64)
        assert not oracle.supports_k(t, 256) and not oracle.supports_k_row(t, 256)
    assert oracle.supports(Q3_K, 256) and oracle.supports_k(Q3_K, 2048) and not oracle.supports_k_row(Q3_K, 896)
    assert not oracle.supports_flat(Q3_K, 2048)   # vecdot.rs:4082, 4593-4594
    assert oracle.supports(Q5_K, 256) and oracle.supports_k(Q5_K, 512) and oracle.supports_k_row(Q5_K, 768)
    assert not oracle.supports(Q5_K, 128) and not oracle.supports_flat(Q5_K, 256)
    assert oracle.supports_k(Q6_K, 256) and not oracle.supports_k(Q8_0, 256)
    assert oracle.supports_k_row(Q4_K, 256) and not oracle.supports_k_row(Q4_K, 128)
    assert oracle.supports_flat(Q8_0, 32) and not oracle.supports_flat(Q4_K, 256)
    assert not oracle.supports(0, 256)


def test_block_sums_entry_matches_per_row_calls():
    in_dim, out_dim, T = 512, 3, 2
    raw, x = k_fixture(Q4_K, in_dim, out_dim, T, 12)
    isum, imin = oracle.block_sums(Q4_K, raw, in_dim, out_dim, x, T)
    rb = row_bytes(Q4_K, in_dim)
    for t in range(T):
        act = oracle.quantize_act_k_row(x[t * in_dim:(t + 1) * in_dim])
        for o in range(out_dim):
            _, a, b = oracle.dot_k_row(Q4_K, raw[o * rb:(o + 1) * rb], act, want_sums=True)
            assert np.array_equal(isum[t, o], a) and np.array_equal(imin[t, o], b)


def test_q5_k_unpack_applies_the_high_bit_to_every_sub_block():
    """vecdot.rs:4141-4165: every qh bit set and every nibble zero: every unpacked weight is exactly
    16 on the decode path and on the K-GEMM path.  With all-one activations quantized to 127 each
    sub-block's dot is 32 * 16 * 127 and the scales are 1."""
    block = np.zeros(176, np.uint8)
    block[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    block[4:16] = [1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]
    block[16:48] = 0xFF
    x = np.ones(256, np.float32)
    act = oracle.quantize_act_k_row(x)
    v, isum, imin = oracle.dot_k_row(Q5_K, block, act, want_sums=True)
    assert isum[0] == 8 * 32 * 16 * 127 and imin[0] == 0
    assert v == np.float32(act[1][0] * np.float32(np.float32(1.0) * np.float32(isum[0])))
    got = oracle.k_gemm_t(Q5_K, block, 256, 1, x, 1)
    assert got[0, 0] == np.float32(act[1][0] * np.float32(isum[0]))


def test_q3_k_unpack_applies_the_inverted_high_bit():
    """vecdot.rs:3938-3968 through the decode path and the K-GEMM path: with every 2-bit field 0,
    hmask clear makes every weight -4 and hmask set makes it 0.  Scale bytes 0x20 unpack to
    0 x 8, 34 x 4, 2 x 4 (minus 32); all-one activations quantize to 127."""
    x = np.ones(256, np.float32)
    act = oracle.quantize_act_k_row(x)
    for hmask, w in ((0x00, -4), (0xFF, 0)):
        block = np.zeros(110, np.uint8)
        block[0:32] = hmask
        block[96:108] = 0x20
        block[108:110] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
        v, isum, _ = oracle.dot_k_row(Q3_K, block, act, want_sums=True)
        assert isum[0] == (8 * (0 - 32) + 4 * (34 - 32) + 4 * (2 - 32)) * 16 * w * 127
        assert v == np.float32(np.float32(act[1][0] * np.float32(1.0)) * np.float32(isum[0]))
        got = oracle.k_gemm_t(Q3_K, block, 256, 1, x, 1)
        assert got[0, 0] == np.float32(act[1][0] * np.float32(np.float32(1.0) * np.float32(isum[0])))


def test_iq4_nl_block_unpack_is_exact_for_every_byte_value():
    """vecdot.rs:3866-3887: all 256 byte values in every position against the table."""
    table = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.int8)
    for base in range(256):
        qs = ((base + 17 * np.arange(16)) % 256).astype(np.uint8)
        _, w = oracle.unpack_flat_block(IQ4_NL, np.concatenate([np.zeros(2, np.uint8), qs]))
        assert np.array_equal(w, np.concatenate([table[qs & 15], table[qs >> 4]])), base


def test_q4_0_uses_its_own_zero_point_not_q5_0s():
    """vecdot.rs:4226-4237: all-zero nibbles unpack to -8 for Q4_0 and to -16 for Q5_0."""
    one = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    dw, w = oracle.unpack_flat_block(Q4_0, np.concatenate([one, np.zeros(16, np.uint8)]))
    assert dw == 1.0 and np.all(w == -8)
    dw, w = oracle.unpack_flat_block(Q5_0, np.concatenate([one, np.zeros(20, np.uint8)]))
    assert dw == 1.0 and np.all(w == -16)
    dw, w = oracle.unpack_flat_block(Q5_0, np.concatenate([one, np.full(4, 0xFF, np.uint8), np.full(16, 0xFF, np.uint8)]))
    assert np.all(w == 15)


@pytest.mark.parametrize("ggml_type", [Q5_0, Q4_0, IQ4_NL])
def test_flat32_row_and_gemm_are_left_to_right_f32_over_independent_integer_sums(ggml_type):
    """dot_q5_0 / _q4_0 / _iq4_nl: total += dw * act.d[b] * isum (vecdot.rs:2842-2883) and the flat
    GEMM's acc += d * s * isum (vecdot.rs:2618-2624) rebuilt in numpy f32 from an independent decode;
    matmul_decode rows equal single-token results."""
    f = np.float32
    in_dim, out_dim, T = 896, 5, 6
    raw, x = k_fixture(ggml_type, in_dim, out_dim, T, 21)
    rb = row_bytes(ggml_type, in_dim)
    gemm = oracle.matmul(ggml_type, raw, in_dim, out_dim, x, T).reshape(T, out_dim)
    dec = oracle.matmul_decode(ggml_type, raw, in_dim, out_dim, x, T).reshape(T, out_dim)
    for o in range(out_dim):
        row = raw[o * rb:(o + 1) * rb]
        _, _, _, dw, _ = np_unpack(ggml_type, row, in_dim)
        for t in range(T):
            act = oracle.quantize_act(x[t * in_dim:(t + 1) * in_dim])
            isum, _ = np_block_sums(ggml_type, row, in_dim, act[0])
            a = b = f(0)
            for blk in range(in_dim // 32):
                a = f(a + f(f(dw[blk] * act[1][blk]) * f(isum[blk])))
                b = f(b + f(f(act[1][blk] * dw[blk]) * f(isum[blk])))
            assert oracle.dot_row(ggml_type, row, act).view(np.uint32) == a.view(np.uint32)
            assert dec[t, o].view(np.uint32) == a.view(np.uint32)
            assert gemm[t, o].view(np.uint32) == b.view(np.uint32)

"""The CPU restatement of Q5_1, Q2_K and IQ4_XS: block decode against ggml's published layouts, the
integer stage against int64 numpy, the f32 order rebuilt from independent integer sums, the budget
against the dequantized reference, and the routing of matmul / matmul_decode."""
import numpy as np
import pytest

import oracle
from helpers import (BLOCK, IQ4_XS, Q2_K, Q5_1, activations, activations_t, fixture_row, k_fixture, pin_scales,
                     pseudo_bytes_fast, row_bytes)

KVALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.int64)
f = np.float32


def f16_at(blocks, off):
    return blocks[:, off:off + 2].copy().view(np.float16).astype(np.float32).reshape(-1)


def np_decode(t, row):
    """Independent numpy decode of a row.  Returns (q int64 [n], integer scale per element [n], integer
    min per element [n] or None, d [blocks], second f16 field [blocks] or None)."""
    bb, _ = BLOCK[t]
    blocks = row.reshape(-1, bb)
    nb = blocks.shape[0]
    if t == Q5_1:    # d | m | qh:u32 | qs[16]: elements 0..16 low nibbles, 16..32 high, fifth bit e of qh (quant.rs:615-636)
        qs = blocks[:, 8:].astype(np.int64)
        bits = np.unpackbits(blocks[:, 4:8].copy(), axis=1, bitorder="little").astype(np.int64)
        q = np.concatenate([qs & 15, qs >> 4], axis=1) + 16 * bits
        return q.reshape(-1), None, None, f16_at(blocks, 0), f16_at(blocks, 2)
    if t == IQ4_XS:  # d | scales_h:u16 | scales_l[4] | qs[128]; sub-block ib: 16 bytes, low nibbles first (quant.rs:1350-1375)
        sh = blocks[:, 2].astype(np.int64) | (blocks[:, 3].astype(np.int64) << 8)
        sl = blocks[:, 4:8].astype(np.int64)
        ls = np.empty((nb, 8), np.int64)
        for ib in range(8):
            ls[:, ib] = (((sl[:, ib // 2] >> (4 * (ib % 2))) & 15) | (((sh >> (2 * ib)) & 3) << 4)) - 32
        qs = blocks[:, 8:].astype(np.int64).reshape(nb, 8, 16)
        q = KVALUES[np.concatenate([qs & 15, qs >> 4], axis=2)]
        return q.reshape(-1), np.repeat(ls, 32, axis=1).reshape(-1), None, f16_at(blocks, 0), None
    # Q2_K: scales[16] (low nibble scale, high nibble min, one per 16) | qs[64] | d | dmin; group 2p + half takes
    # qs[32 (p / 4) + 16 half + l] >> 2 (p % 4) (quant.rs:798-827)
    sc = blocks[:, 0:16].astype(np.int64)
    qs = blocks[:, 16:80].astype(np.int64).reshape(nb, 2, 32)
    q = np.empty((nb, 8, 32), np.int64)
    for p in range(8):
        q[:, p, :] = (qs[:, p // 4, :] >> (2 * (p % 4))) & 3
    return (q.reshape(-1), np.repeat(sc & 15, 16, axis=1).reshape(-1), np.repeat(sc >> 4, 16, axis=1).reshape(-1),
            f16_at(blocks, 80), f16_at(blocks, 82))


@pytest.mark.parametrize("t", [Q5_1, Q2_K, IQ4_XS])
def test_dequantize_equals_the_independent_decode(t):
    """value = d * q + m (Q5_1), d * sc * q - dmin * mn (Q2_K), (d * ls) * level (IQ4_XS) in the reference's
    f32 association, over random payloads."""
    bb, be = BLOCK[t]
    n = 4 * be if be == 256 else 16 * be
    row = pin_scales(pseudo_bytes_fast(n // be * bb, 5), t)
    q, sce, mne, d, d2 = np_decode(t, row)
    got = oracle.dequantize(t, row, n)
    de, d2e = np.repeat(d, be), (np.repeat(d2, be) if d2 is not None else None)
    if t == Q5_1:
        want = q.astype(f) * de + d2e
    elif t == IQ4_XS:
        want = (de * sce.astype(f)) * q.astype(f)
    else:
        want = (de * sce.astype(f)) * q.astype(f) - d2e * mne.astype(f)
    assert np.array_equal(got.view(np.uint32), want.astype(f).view(np.uint32))


def test_block_layouts_and_predicates():
    """quant.rs:132-169; vecdot.rs:274-283, 1821-1826, 3083-3093, 2456-2461 and the asymmetry pinned at :4067-4069."""
    assert oracle.tensor_byte_size(Q5_1, 64) == 2 * 24 and oracle.tensor_byte_size(Q2_K, 512) == 2 * 84
    assert oracle.tensor_byte_size(IQ4_XS, 512) == 2 * 136
    assert oracle.supports(Q5_1, 896) and not oracle.supports(Q5_1, 24)
    assert not oracle.supports_k(Q5_1, 2048) and not oracle.supports_k_row(Q5_1, 2048) and not oracle.supports_flat(Q5_1, 896)
    assert oracle.supports(Q2_K, 2048) and not oracle.supports(Q2_K, 896)
    assert oracle.supports_k_row(Q2_K, 2048) and not oracle.supports_k(Q2_K, 2048) and not oracle.supports_flat(Q2_K, 2048)
    assert oracle.supports(IQ4_XS, 2048) and oracle.supports_k(IQ4_XS, 2048) and oracle.supports_k_row(IQ4_XS, 2048)
    assert not oracle.supports(IQ4_XS, 896) and not oracle.supports_flat(IQ4_XS, 2048)


@pytest.mark.parametrize("in_dim", [256, 2048])
@pytest.mark.parametrize("t", [Q2_K, IQ4_XS])
def test_k_row_sums_and_float_order(t, in_dim):
    """dot_k_row_iq4_xs (vecdot.rs:3245-3266): isum = sum_ib ls * dot32, total += act.d * d * isum, left to right;
    dot_k_row_q2_k (:3296-3318): isum over the groups' scales, imin over their mins against the per-16
    activation sums, total += act.d * (d * isum - dmin * imin)."""
    row = fixture_row(t, in_dim, 9)
    act = oracle.quantize_act_k_row(activations(in_dim))
    got, isum, imin = oracle.dot_k_row(t, row, act, want_sums=True)
    q, sce, mne, d, dmin = np_decode(t, row)
    xq = act[0].astype(np.int64)
    wi = (q * sce * xq).reshape(-1, 256).sum(axis=1)
    assert np.array_equal(isum, wi)
    total = f(0)
    if t == Q2_K:
        wm = (mne * xq).reshape(-1, 256).sum(axis=1)
        assert np.array_equal(imin, wm)
        for s in range(in_dim // 256):
            total = f(total + f(act[1][s] * f(f(d[s] * f(wi[s])) - f(dmin[s] * f(wm[s])))))
    else:
        for s in range(in_dim // 256):
            total = f(total + f(f(act[1][s] * d[s]) * f(wi[s])))
    assert np.float32(got).view(np.uint32) == np.float32(total).view(np.uint32)


@pytest.mark.parametrize("in_dim", [32, 896, 4864])
def test_q5_1_row_sums_and_float_order(in_dim):
    """dot_q5_1 (vecdot.rs:2886-2899): total += act.d[b] * (dw * isum + m * block_sum), blocks ascending."""
    row = fixture_row(Q5_1, in_dim, 3)
    act = oracle.quantize_act(activations(in_dim))
    q, _, _, d, m = np_decode(Q5_1, row)
    xq = act[0].astype(np.int64)
    wi = (q * xq).reshape(-1, 32).sum(axis=1)
    bs = xq.reshape(-1, 32).sum(axis=1)
    total = f(0)
    for b in range(in_dim // 32):
        total = f(total + f(act[1][b] * f(f(d[b] * f(wi[b])) + f(m[b] * f(bs[b])))))
    got = oracle.dot_row(Q5_1, row, act)
    assert np.float32(got).view(np.uint32) == np.float32(total).view(np.uint32)
    # the rows-unpacked-once form (scale * isum - (-m) * bsum, vecdot.rs:1302-1314, 1698) has the same bits
    other = f(0)
    for b in range(in_dim // 32):
        other = f(other + f(act[1][b] * f(f(d[b] * f(wi[b])) - f(f(-m[b]) * f(bs[b])))))
    assert np.float32(other).view(np.uint32) == np.float32(total).view(np.uint32)


@pytest.mark.parametrize("in_dim", [256, 2048])
def test_q2_k_unpacked_form_float_order(in_dim):
    """unpack_q2_k + dot_unpacked (vecdot.rs:1144-1164, 420-425): per-32 activations, per group of 16
    total += act.d[g / 2] * ((d * sc) * isum_g - (dmin * mn) * sums[g]), groups ascending."""
    row = fixture_row(Q2_K, in_dim, 4)
    act = oracle.quantize_act(activations(in_dim))
    q, sce, mne, d, dmin = np_decode(Q2_K, row)
    xq = act[0].astype(np.int64)
    ig = (q * xq).reshape(-1, 16).sum(axis=1)
    assert np.array_equal(act[2], xq.reshape(-1, 16).sum(axis=1))
    total = f(0)
    for g in range(in_dim // 16):
        s = g // 16
        scale, mn = f(d[s] * f(sce[16 * g])), f(dmin[s] * f(mne[16 * g]))
        total = f(total + f(act[1][g // 2] * f(f(scale * f(ig[g])) - f(mn * f(act[2][g])))))
    got = oracle.dot_unpacked_q2_k(row, act)
    assert np.float32(got).view(np.uint32) == np.float32(total).view(np.uint32)


@pytest.mark.parametrize("t,in_dim", [(Q5_1, 32), (Q5_1, 896), (Q5_1, 4864), (Q2_K, 256), (Q2_K, 2048), (Q2_K, 5632),
                                      (IQ4_XS, 256), (IQ4_XS, 2048), (IQ4_XS, 5632)])
@pytest.mark.parametrize("seed", [1, 7, 99])
def test_decode_dots_match_the_dequantized_reference(t, in_dim, seed):
    """vecdot.rs:3436-3526 `check` (Q5_1: :4187-4189, budget 0.01) and :4011-4040 (per-256 decode, budget 0.02):
    |got - sum w x| <= budget * sum |w x| with w = dequantize(row)."""
    row = fixture_row(t, in_dim, seed)
    x = activations(in_dim)
    w = oracle.dequantize(t, row, in_dim).astype(np.float64)
    ref, mag = (w * x).sum(), np.abs(w * x).sum()
    if t == Q5_1:
        got, budget = oracle.dot_row(t, row, oracle.quantize_act(x)), 0.01
    else:
        got, budget = oracle.dot_k_row(t, row, oracle.quantize_act_k_row(x)), 0.02
    assert abs(float(got) - ref) <= budget * max(mag, 1e-6)
    if t == Q2_K:
        got2 = oracle.dot_unpacked_q2_k(row, oracle.quantize_act(x))
        assert abs(float(got2) - ref) <= 0.01 * max(mag, 1e-6)


def test_iq4_xs_gemm_order_and_batch_independence():
    """gemm_k_iq4_xs = accumulate_sym32 alone (vecdot.rs:2271-2322): acc += ad * (d * isum) per super-block, from
    independent integer sums; and the same bits whatever the batch (vecdot.rs:4522-4549)."""
    in_dim, out_dim, T = 1024, 3, 7
    raw, x = k_fixture(IQ4_XS, in_dim, out_dim, T, 31)
    got = oracle.k_gemm_t(IQ4_XS, raw, in_dim, out_dim, x, T)
    rb = row_bytes(IQ4_XS, in_dim)
    for o in range(out_dim):
        q, sce, _, d, _ = np_decode(IQ4_XS, raw[o * rb:(o + 1) * rb])
        for t in range(T):
            act = oracle.quantize_act_k_row(x[t * in_dim:(t + 1) * in_dim])
            wi = (q * sce * act[0].astype(np.int64)).reshape(-1, 256).sum(axis=1)
            acc = f(0)
            for s in range(in_dim // 256):
                acc = f(acc + f(act[1][s] * f(d[s] * f(wi[s]))))
            assert np.float32(got[o, t]).view(np.uint32) == np.float32(acc).view(np.uint32)
    for n in (2, 3, 5):
        part = oracle.k_gemm_t(IQ4_XS, raw, in_dim, out_dim, x[: n * in_dim], n)
        assert np.array_equal(part.view(np.uint32), got[:, :n].view(np.uint32))


@pytest.mark.parametrize("t", [Q5_1, Q2_K, IQ4_XS])
def test_matmul_routing(t):
    """cpu.rs:55-167: one token takes dot_k_row where supports_k_row (Q2_K, IQ4_XS) and dot_row otherwise (Q5_1);
    several tokens take the K GEMM (IQ4_XS) or the rows-unpacked-once path over per-32 activations (Q5_1, Q2_K);
    matmul_decode (cpu.rs:265-317) is the one-token arithmetic per row of the batch."""
    in_dim, out_dim, T = 512, 5, 6
    raw = pin_scales(pseudo_bytes_fast(row_bytes(t, in_dim) * out_dim, 21), t)
    x = np.concatenate([activations_t(in_dim, k) for k in range(T)])
    rb = row_bytes(t, in_dim)
    one = oracle.matmul(t, raw, in_dim, out_dim, x[:in_dim], 1)
    many = oracle.matmul(t, raw, in_dim, out_dim, x, T)
    dec = oracle.matmul_decode(t, raw, in_dim, out_dim, x, T)
    for o in range(out_dim):
        row = raw[o * rb:(o + 1) * rb]
        for k in range(T):
            xs = x[k * in_dim:(k + 1) * in_dim]
            if t == Q5_1:
                single = multi = oracle.dot_row(t, row, oracle.quantize_act(xs))
            elif t == Q2_K:
                single = oracle.dot_k_row(t, row, oracle.quantize_act_k_row(xs))
                multi = oracle.dot_unpacked_q2_k(row, oracle.quantize_act(xs))
            else:
                single = oracle.dot_k_row(t, row, oracle.quantize_act_k_row(xs))
                multi = oracle.k_gemm_t(t, row, in_dim, 1, xs, 1)[0, 0]
            assert np.float32(dec[k, o]).view(np.uint32) == np.float32(single).view(np.uint32)
            assert np.float32(many[k, o]).view(np.uint32) == np.float32(multi).view(np.uint32)
            if k == 0:
                assert np.float32(one[0, o]).view(np.uint32) == np.float32(single).view(np.uint32)


def test_scalar_and_vector_builds_agree_on_the_new_types():
    for t, in_dim in ((Q5_1, 896), (Q2_K, 1024), (IQ4_XS, 1024)):
        raw = pin_scales(pseudo_bytes_fast(row_bytes(t, in_dim) * 4, 8), t)
        x = np.concatenate([activations_t(in_dim, k) for k in range(5)])
        a = [oracle.matmul(t, raw, in_dim, 4, x, 5), oracle.matmul_decode(t, raw, in_dim, 4, x, 5)]
        oracle.force_scalar(True)
        try:
            b = [oracle.matmul(t, raw, in_dim, 4, x, 5), oracle.matmul_decode(t, raw, in_dim, 4, x, 5)]
        finally:
            oracle.force_scalar(False)
        for u, v in zip(a, b):
            assert np.array_equal(u.view(np.uint32), v.view(np.uint32))


def test_q5_1_min_term_is_added_not_subtracted():
    """vecdot.rs:4195-4218: with d = 0 the quantized term vanishes and every weight is exactly m = 2.5 -- a sign
    slip would bias every weight by 2m.  The fused dot of that block against x is then 2.5 * sum(q_x) * scale_x, and
    through matmul at several tokens (the rows-unpacked-once path, where the min enters as -2.5) the same value."""
    block = np.concatenate([np.frombuffer(np.float16(0.0).tobytes(), np.uint8), np.frombuffer(np.float16(2.5).tobytes(), np.uint8),
                            np.zeros(4, np.uint8), np.zeros(16, np.uint8)])
    assert np.all(np.abs(oracle.dequantize(Q5_1, block, 32) - 2.5) < 1e-6)
    x = activations(32)
    q, d, _ = oracle.quantize_act(x)
    want = f(2.5) * d[0] * f(q.astype(np.int64).sum())
    got1 = oracle.matmul(Q5_1, block, 32, 1, x, 1)[0]
    assert abs(got1 - want) <= 1e-6 * max(1.0, abs(want)), (got1, want)
    got3 = oracle.matmul(Q5_1, block, 32, 1, np.concatenate([x, x, x]), 3).reshape(-1)
    assert np.all(np.abs(got3 - want) <= 1e-5 * max(1.0, abs(want))), (got3, want)

"""Pins the oracle's activation quantizers (engine/vecdot.rs:95-126, 3030-3053, 1858-1910,
2483-2525) against the reference's own quantizer tests (vecdot.rs:4259-4410) and against an
independent numpy formulation.  CPU only."""
import numpy as np
import pytest

import oracle


def adversarial_blocks() -> np.ndarray:
    """vecdot.rs:4274-4344 quantize_act_adversarial_blocks, block for block."""
    f = np.float32
    blocks = []
    blocks.append(np.zeros(32, f))

    ties = np.full(32, 254.0, f)
    half_down = np.nextafter(f(0.5), f(0.0))
    for i in range(1, 32):
        ties[i] = {1: f(1.0), 2: f(-1.0), 3: f(3.0), 4: f(-3.0), 5: f(2.0) * half_down,
                   6: f(-2.0) * half_down}.get(i % 8, f(5.0))
    blocks.append(ties)

    tiny = np.full(32, np.finfo(f).tiny, f)
    tiny[0] = f(1.0e30)
    tiny[7] = -np.frombuffer(np.uint32(1).tobytes(), f)[0]
    tiny[9] = np.frombuffer(np.uint32(1).tobytes(), f)[0]
    blocks.append(tiny)

    nans = np.full(32, 4.0, f)
    nans[0] = np.nan
    nans[3] = -np.nan
    nans[31] = np.nan
    blocks.append(nans)

    infs = np.full(32, 1.0, f)
    infs[5] = np.inf
    infs[6] = -np.inf
    blocks.append(infs)

    neg = np.full(32, 0.25, f)
    neg[13] = -100.0
    neg[20] = -60.0
    blocks.append(neg)

    lcg = 0x12345678
    spread = np.zeros(32, f)
    for i in range(32):
        lcg = (lcg * 1664525 + 1013904223) & 0xFFFFFFFF
        spread[i] = f(lcg >> 8) / f(8388608.0) - f(0.5)
    spread[0], spread[1] = 1.0, -1.0
    blocks.append(spread)
    return np.concatenate(blocks)


def numpy_quantize(x: np.ndarray, group: int):
    """Independent formulation of the quantizer rule (NaN-blind |max|, scale = amax/127,
    multiply by 1/scale, round half away from zero, NaN -> 0, clamp to +-127), vectorised and
    with rounding written as trunc + exact fractional test instead of roundf."""
    f = np.float32
    x = x.astype(f).reshape(-1, group)
    with np.errstate(all="ignore"):
        a = np.abs(x)
        amax = np.where(np.isnan(a), f(0), a).max(axis=1).astype(f)
        scale = (amax / f(127.0)).astype(f)
        inv = np.where(scale > 0, f(1.0) / scale, f(0.0)).astype(f)
        y = (x * inv[:, None]).astype(f)
        t = np.trunc(y)
        frac = np.abs(y - t)  # exact in f32
        r = np.where(frac >= f(0.5), t + np.sign(y), t)
        r = np.where(np.isnan(r), f(0), r)
        q = np.clip(r, -127, 127).astype(np.int8)
    return q.reshape(-1), scale


def test_quantize_act_handles_an_all_zero_block_without_nan():
    """vecdot.rs:4259-4264."""
    q, d, s = oracle.quantize_act(np.zeros(64, np.float32))
    assert np.all(d == 0.0) and np.all(q == 0) and np.all(s == 0)


def test_quantize_act_rounds_ties_away_from_zero_like_f32_round():
    """vecdot.rs:4395-4410."""
    x = np.full(32, 254.0, np.float32)
    x[1], x[2], x[3], x[4] = 1.0, 3.0, -1.0, -3.0
    q, d, _ = oracle.quantize_act(x)
    assert (q[1], q[2], q[3], q[4]) == (1, 2, -1, -2)
    assert d[0] == np.float32(2.0)


def test_quantize_act_adversarial_blocks_by_hand():
    """Expected bytes derived by hand from the rule for each block of vecdot.rs:4274-4344 (the
    reference compares its vector kernel with its scalar definition on these; here the scalar
    definition's outputs are written out)."""
    x = adversarial_blocks()
    q, d, sums = oracle.quantize_act(x)
    q = q.reshape(7, 32)
    # 0: zeros
    assert np.all(q[0] == 0) and d[0] == 0.0
    # 1: ties, inv == 0.5 exactly
    want = np.empty(32, np.int8)
    want[0] = 127
    for i in range(1, 32):
        want[i] = {1: 1, 2: -1, 3: 2, 4: -2, 5: 0, 6: 0}.get(i % 8, 3)
    assert np.array_equal(q[1], want) and d[1] == np.float32(2.0)
    # 2: 1e30 against denormals: everything else underflows to 0
    assert q[2][0] == 127 and np.all(q[2][1:] == 0)
    assert d[2] == np.float32(1.0e30) / np.float32(127.0)
    # 3: NaN skipped by the max fold (amax = 4), NaN lanes -> 0, 4.0 -> 127
    want = np.full(32, 127, np.int8)
    want[[0, 3, 31]] = 0
    assert np.array_equal(q[3], want) and d[3] == np.float32(4.0) / np.float32(127.0)
    # 4: infinity: scale = inf, inv = 0, finite -> 0, inf*0 = NaN -> 0
    assert np.all(q[4] == 0) and np.isinf(d[4]) and d[4] > 0
    # 5: the maximum is negative
    want = np.zeros(32, np.int8)
    want[13], want[20] = -127, -76
    assert np.array_equal(q[5], want) and d[5] == np.float32(100.0) / np.float32(127.0)
    # 6: the LCG spread lies in [-0.5, 1.5), so lanes 0/1 (+-1) are symmetric but not extreme
    wq, wd = numpy_quantize(x[6 * 32:], 32)
    assert np.array_equal(q[6], wq) and d[6] == wd[0] and q[6][0] == -q[6][1] and q[6].max() == 127
    # per-16 sums are the sums of the bytes written (vecdot.rs:4383-4390)
    assert np.array_equal(sums, q.reshape(-1, 16).astype(np.int32).sum(axis=1))


@pytest.mark.parametrize("group,fn", [(32, "quantize_act"), (256, "quantize_act_k_row")])
def test_quantizers_match_independent_numpy_formulation(group, fn):
    rng = np.random.default_rng(11)
    pieces = [rng.standard_normal(4096).astype(np.float32) * np.float32(3.0),
              (rng.integers(-254, 255, 2048) * 0.5).astype(np.float32),  # many exact ties
              np.tile(adversarial_blocks(), 8)[:1792]]
    x = np.concatenate(pieces)
    x = x[: x.size // 256 * 256]
    q, d, s = getattr(oracle, fn)(x)
    wq, wd = numpy_quantize(x, group)
    assert np.array_equal(q, wq)
    assert np.array_equal(d.view(np.uint32), wd.view(np.uint32))
    assert np.array_equal(s, wq.reshape(-1, 16).astype(np.int32).sum(axis=1))


def test_k_row_scale_is_per_256_not_per_32():
    """vecdot.rs:3030-3053: one scale per super-block; a block whose own maximum is smaller than
    the super-block's is quantized against the larger one."""
    x = np.zeros(512, np.float32)
    x[0] = 127.0
    x[40] = 63.5  # block 1 of super-block 0: per-32 would give 127, per-256 gives round(63.5)=64
    x[300] = 2.0
    q, d, _ = oracle.quantize_act_k_row(x)
    assert d.size == 2 and d[0] == np.float32(1.0) and d[1] == np.float32(2.0) / np.float32(127.0)
    assert q[0] == 127 and q[40] == 64 and q[300] == 127
    q32, d32, _ = oracle.quantize_act(x)
    assert q32[40] == 127 and d32[1] == np.float32(0.5)


@pytest.mark.parametrize("n_tokens", [1, 4, 7])
def test_act_q8k_is_the_k_row_quantizer_tiled_by_four_tokens(n_tokens):
    """vecdot.rs:1858-1910: same per-256 arithmetic; q[tile][block][token][32], d[tile][super]
    [token], bsum[tile][super][token][8] = per-32 sums; padding tokens stay zero."""
    in_dim = 512
    rng = np.random.default_rng(5)
    x = rng.standard_normal((n_tokens, in_dim)).astype(np.float32)
    q, d, b = oracle.act_q8k_quantize(x, in_dim, n_tokens)
    for t in range(4 * q.shape[0]):
        tl, k = divmod(t, 4)
        if t >= n_tokens:
            assert not q[tl, :, k].any() and not d[tl, :, k].any() and not b[tl, :, k].any()
            continue
        rq, rd, rs = oracle.quantize_act_k_row(x[t])
        assert np.array_equal(q[tl, :, k, :].reshape(-1), rq)
        assert np.array_equal(d[tl, :, k].view(np.uint32), rd.view(np.uint32))
        assert np.array_equal(b[tl, :, k, :].reshape(-1).astype(np.int32),
                              rs.reshape(-1, 2).sum(axis=1))


@pytest.mark.parametrize("n_tokens", [1, 5])
def test_act_q8flat_is_the_per_32_quantizer_tiled(n_tokens):
    """vecdot.rs:2483-2525."""
    in_dim = 96
    rng = np.random.default_rng(6)
    x = rng.standard_normal((n_tokens, in_dim)).astype(np.float32)
    q, d = oracle.act_q8flat_quantize(x, in_dim, n_tokens)
    for t in range(n_tokens):
        tl, k = divmod(t, 4)
        rq, rd, _ = oracle.quantize_act(x[t])
        assert np.array_equal(q[tl, :, k, :].reshape(-1), rq)
        assert np.array_equal(d[tl, :, k].view(np.uint32), rd.view(np.uint32))

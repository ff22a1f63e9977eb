"""The kernel that takes 2 to 16 tokens over a Q6_K matrix of many rows in one streaming pass on the matrix
cores (`ogm_gemm_ft_q6k_kernel`): bit for bit against the CPU restatement in both float orders -- matmul of
several tokens (gemm_k_q6_k, vecdot.rs:2352-2398) and decode batches (dot_k_row_q6_k per token,
vecdot.rs:3215-3241, cpu.rs:265-317) -- at ragged row counts, every token count, the extremes of the integer
range, through grouped calls, and at the vocabulary projection's full size where it is the default."""
import numpy as np
import pytest

import oracle
from helpers import Q4_K, Q6_K, activations_t, pin_scales, pseudo_bytes_fast, row_bytes, synth_weights, synth_x

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def be():
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()  # raises if the HIP library or the device is missing: no fallback
    b.set_tuning("gemm_few_tokens_min_rows", 1)   # whatever the row count
    yield b
    b.close()


def qm(raw, t, in_dim, out_dim):
    from orangu_amd import QuantMatrix
    return QuantMatrix(np.ascontiguousarray(raw), t, in_dim, out_dim)


def assert_bits(got, want, what):
    got = np.asarray(got, np.float32).reshape(-1)
    want = np.asarray(want, np.float32).reshape(-1)
    same = got.view(np.uint32) == want.view(np.uint32)
    assert same.all(), f"{what}: {(~same).sum()} of {got.size} differ in bits; first at " \
                       f"{np.nonzero(~same)[0][:5]} got {got[~same][:5]} want {want[~same][:5]}"


def kernel_for(T):
    return "ogm_gemm_ft_q6k_kernel" if T <= 8 else "ogm_gemm_ft_q6k_t16_kernel"


@pytest.mark.parametrize("in_dim,out_dim", [(1024, 1), (1024, 31), (1024, 129), (2048, 300), (4096, 530), (14336, 70)])
@pytest.mark.parametrize("T", [2, 3, 4, 5, 7, 8, 9, 12, 16])
def test_both_float_orders_are_bit_exact(be, in_dim, out_dim, T):
    raw = synth_weights(Q6_K, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T + 11)
    w = qm(raw, Q6_K, in_dim, out_dim)
    say("few tokens", in_dim, out_dim, T)
    fits = in_dim * (8 if T <= 8 else 16) <= 150 * 1024
    got = be.matmul(x, T, w)
    assert (be.last_kernel() == kernel_for(T)) == fits, be.last_kernel()
    assert_bits(got, oracle.matmul(Q6_K, raw, in_dim, out_dim, x, T), "matmul")
    got = be.matmul_decode(x, T, w)
    assert (be.last_kernel() == kernel_for(T)) == fits, be.last_kernel()
    assert_bits(got, oracle.matmul_decode(Q6_K, raw, in_dim, out_dim, x, T), "decode batch")


@pytest.mark.parametrize("T", [2, 8, 16])
def test_extreme_integer_sums_are_exact(be, T):
    """Every weight at one end of its range under the largest scales, every activation at +-127: the
    per-group products reach 16 * 127 * 32 and a super-block's sum 1.3e8."""
    in_dim, out_dim = 2048, 96
    for fill, scale in ((0xFF, 0x7F), (0x00, 0x80), (0xFF, 0x80)):
        blk = np.zeros(210, np.uint8)
        blk[:192] = fill
        blk[192:208] = scale
        blk[208:210] = np.frombuffer(np.float16(0.001).tobytes(), np.uint8)
        raw = np.tile(blk, (in_dim // 256) * out_dim)
        w = qm(raw, Q6_K, in_dim, out_dim)
        for sign in (1.0, -1.0):
            x = np.full(T * in_dim, sign * 3.0, np.float32)
            got = be.matmul(x, T, w)
            assert be.last_kernel() == kernel_for(T)
            assert_bits(got, oracle.matmul(Q6_K, raw, in_dim, out_dim, x, T), f"extreme {fill:#x} {scale:#x} {sign}")
            isum, _ = be.dump_block_sums(x[:in_dim], 1, w)
            assert np.abs(isum).max() >= 16 * 16 * 127 * 31 * 127


def test_random_bytes_and_special_activations(be):
    """Weights of arbitrary bytes (scales pinned finite) and activations with a row of zeros, a row of denormals and a NaN."""
    in_dim, out_dim, T = 1024, 200, 6
    raw = pin_scales(pseudo_bytes_fast(row_bytes(Q6_K, in_dim) * out_dim, 77), Q6_K)
    x = np.concatenate([activations_t(in_dim, k) for k in range(T)])
    x[in_dim:2 * in_dim] = 0.0
    x[2 * in_dim:3 * in_dim] = np.float32(1e-42)
    x[3 * in_dim + 5] = np.nan   # quantizes to 0 and leaves the row's scale alone (vecdot.rs:3030-3053)
    w = qm(raw, Q6_K, in_dim, out_dim)
    for fn, ref in ((be.matmul, oracle.matmul), (be.matmul_decode, oracle.matmul_decode)):
        got = fn(x, T, w)
        assert be.last_kernel() == kernel_for(T)
        assert_bits(got, ref(Q6_K, raw, in_dim, out_dim, x, T), fn.__name__)


def test_grouped_calls_and_other_types_keep_their_kernels(be):
    """matmul_batch over Q6_K matrices that share their input launches the kernel once per matrix; a Q4_K matrix
    and a single token stay where they were."""
    from orangu_amd import MatmulOp
    in_dim, T = 1024, 4
    x = synth_x(T, in_dim, seed=5)
    raws = [synth_weights(Q6_K, in_dim, o, seed=o) for o in (40, 129)]
    ws = [qm(r, Q6_K, in_dim, o) for r, o in zip(raws, (40, 129))]
    ys = be.matmul_batch([MatmulOp(x, T, w) for w in ws])
    assert be.last_kernel() == kernel_for(T)
    for y, r, o in zip(ys, raws, (40, 129)):
        assert_bits(y, oracle.matmul(Q6_K, r, in_dim, o, x, T), f"grouped {o}")
    raw4 = synth_weights(Q4_K, in_dim, 64, seed=9)
    be.matmul(x, T, qm(raw4, Q4_K, in_dim, 64))
    assert not be.last_kernel().startswith("ogm_gemm_ft")
    be.matmul(np.asarray(x).reshape(-1)[:in_dim], 1, ws[0])
    assert not be.last_kernel().startswith("ogm_gemm_ft")


def test_default_routing_takes_it_for_the_vocabulary_projection_only():
    """Without the tuning key: 4096 -> 128256 and 4096 -> 32000 at 3 to 16 tokens run the kernel, two tokens and
    4096 -> 14336 do not; and the full-size results are bit-exact in both orders (checked on a sample of rows against the oracle over the same
    rows as a smaller matrix -- a row's result does not depend on the others)."""
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()
    try:
        in_dim, out_dim = 4096, 128256
        raw = synth_weights(Q6_K, in_dim, out_dim, seed=3)
        w = qm(raw, Q6_K, in_dim, out_dim)
        rb = row_bytes(Q6_K, in_dim)
        rows = np.r_[0:40, 64000:64040, out_dim - 40:out_dim]
        sub = np.ascontiguousarray(raw.reshape(out_dim, rb)[rows]).reshape(-1)
        for T in (2, 3, 4, 8, 16):
            x = synth_x(T, in_dim, seed=T)
            say("vocabulary projection", T)
            got = b.matmul(x, T, w).reshape(T, out_dim)
            assert (b.last_kernel() == kernel_for(T)) == (T >= 3), b.last_kernel()
            assert_bits(got[:, rows], oracle.matmul(Q6_K, sub, in_dim, len(rows), x, T), f"matmul {T}")
            got = b.matmul_decode(x, T, w).reshape(T, out_dim)
            assert (b.last_kernel() == kernel_for(T)) == (T >= 3), b.last_kernel()
            assert_bits(got[:, rows], oracle.matmul_decode(Q6_K, sub, in_dim, len(rows), x, T), f"decode {T}")
        w32 = qm(raw[:rb * 32000], Q6_K, in_dim, 32000)
        x = synth_x(4, in_dim, seed=2)
        got = b.matmul(x, 4, w32)
        assert b.last_kernel() == kernel_for(4), b.last_kernel()
        assert_bits(np.asarray(got).reshape(4, 32000)[:, :40], oracle.matmul(Q6_K, sub[:rb * 40], in_dim, 40, x, 4), "32000 rows")
        small = qm(synth_weights(Q6_K, 4096, 14336, seed=4), Q6_K, 4096, 14336)
        b.matmul(synth_x(4, 4096, seed=1), 4, small)
        assert not b.last_kernel().startswith("ogm_gemm_ft"), b.last_kernel()
        b.set_tuning("gemm_few_tokens_min_rows", -1)
        b.matmul(synth_x(4, in_dim, seed=1), 4, w)
        assert not b.last_kernel().startswith("ogm_gemm_ft"), b.last_kernel()
    finally:
        b.close()

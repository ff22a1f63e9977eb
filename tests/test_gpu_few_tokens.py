"""GPU parity of the few-token kernel that gives a workgroup one row block of 16 rows (2 to 16 tokens over Q4_K,
Q5_K and Q6_K: the projections of a speculative-decode verify batch, generate.rs:1618-1674, and of a decode
batch, cpu.rs:265-317), through the C ABI against the CPU oracle: every bit of the f32 outputs, in the GEMM's
float order (Backend::matmul at n_tokens > 1) and in the decode dot's (matmul_decode)."""
import sys

import numpy as np
import pytest

import oracle
from helpers import Q4_K, Q5_K, Q6_K, synth_weights, synth_x

pytestmark = pytest.mark.gpu

NAME = {Q4_K: "ogm_gemm_fk_kernel<Q4_K>", Q5_K: "ogm_gemm_fk_kernel<Q5_K>", Q6_K: "ogm_gemm_fk_kernel<Q6_K>"}


@pytest.fixture(scope="module")
def be():
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()  # raises if the HIP library or the device is missing: no fallback
    b.set_tuning("gemm_few_tokens_min_rows", -1)   # keep the many-rows few-token kernel out: this module is about the other one
    b.set_tuning("gemv_mma", 2)                    # from two tokens on for every type (the default leaves Q4_K / Q5_K up to four tokens to the GEMV kernel)
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


@pytest.mark.parametrize("t", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("in_dim,out_dim", [(1024, 40), (2048, 16), (4096, 257), (3072, 100), (14336, 50),
                                            (256, 33), (768, 130), (1536, 70), (2560, 48), (11008, 20)])
@pytest.mark.parametrize("T", [2, 3, 4, 5, 8, 9, 13, 16])
def test_row_block_kernel_matches_cpu_gemm(be, t, in_dim, out_dim, T):
    """One to fifty-six super-blocks a row in every tiling (tiles of 16 rows x 4 blocks, 32 x 2 and 64 x 1, of
    which a workgroup takes 16 rows); row groups that end beyond the matrix; every token count of both slot widths."""
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T)
    got = be.matmul(x, T, qm(raw, t, in_dim, out_dim))
    if (in_dim == 14336 and (T > 8 or t != Q6_K)) or (in_dim == 11008 and T > 8):
        assert not be.last_kernel().startswith("ogm_gemm_fk"), "activations and terms beyond a workgroup's LDS"
    else:
        assert be.last_kernel() == NAME[t]
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), f"type {t} {in_dim}->{out_dim} at {T} tokens")


@pytest.mark.parametrize("t", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("T", [2, 4, 7, 8, 12])
def test_row_block_kernel_in_the_decode_dots_order(be, t, T):
    """matmul_decode over a batch (cpu.rs:265-317): every token's row equals the single-token GEMV's."""
    in_dim, out_dim = 2048, 75
    raw = synth_weights(t, in_dim, out_dim, seed=31 + T)
    x = synth_x(T, in_dim, seed=T + 100)
    w = qm(raw, t, in_dim, out_dim)
    got = be.matmul_decode(x, T, w).reshape(T, out_dim)
    assert be.last_kernel() == NAME[t]
    want = oracle.matmul_decode(t, raw, in_dim, out_dim, x, T).reshape(T, out_dim)
    assert_bits(got, want, f"type {t} decode order at {T} tokens")
    for i in range(T):
        assert_bits(be.matmul(x[i:i + 1], 1, w), want[i], f"token {i} alone")


def test_row_block_kernel_over_several_matrices(be):
    """q / k / v over one input in one launch: the grid runs through the matrices' row blocks in turn."""
    from orangu_amd.hiprt import DeviceBuffer, device_synchronize
    in_dim, T, outs = 1024, 6, (300, 130, 64, 17)
    raws = [synth_weights(Q4_K, in_dim, od, seed=190 + i) for i, od in enumerate(outs)]
    hs = [be.upload_raw(r, Q4_K, in_dim, od) for r, od in zip(raws, outs)]
    x = synth_x(T, in_dim, seed=18)
    xd = DeviceBuffer.from_numpy(x)
    yds = [DeviceBuffer(4 * T * od) for od in outs]
    try:
        be.matmul_multi_dev(hs, xd.ptr, T, [y.ptr for y in yds])
        device_synchronize()
        assert be.last_kernel() == NAME[Q4_K]
        for r, od, yd in zip(raws, outs, yds):
            assert_bits(yd.to_numpy(np.float32, T * od), oracle.matmul(Q4_K, r, in_dim, od, x, T), f"{od} rows of {outs}")
    finally:
        for h in hs:
            be.free_weight(h)
        xd.free()
        for y in yds:
            y.free()


@pytest.mark.parametrize("sign", [1, -1])
def test_row_block_kernel_extreme_integer_ranges(be, sign):
    """The largest magnitudes the integer stage can see: Q4_K nibbles 15 with scales and mins 63, Q5_K with the
    fifth bits set, Q6_K quants 63 (and 0: -32) under scales of +-127 and -128, activations +-127."""
    T, in_dim, rows = 8, 1024, 32
    xe = np.full((T, in_dim), 127.0 * sign, np.float32)
    xe[1::2] *= -1
    xe[:, ::7] = 126.0
    b4 = np.zeros((rows * 4, 144), np.uint8)
    b4[:, 0:2] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    b4[:, 2:4] = np.frombuffer(np.float16(0.02).tobytes(), np.uint8)
    b4[:, 4:] = 0xFF
    b5 = np.zeros((rows * 4, 176), np.uint8)
    b5[:, 0:4] = b4[:, 0:4]
    b5[:, 4:] = 0xFF
    for t, blocks in ((Q4_K, b4), (Q5_K, b5)):
        got = be.matmul(xe, T, qm(blocks.reshape(-1), t, in_dim, rows))
        assert be.last_kernel() == NAME[t]
        assert_bits(got, oracle.matmul(t, blocks.reshape(-1), in_dim, rows, xe, T), f"type {t} extreme ranges")
    for ql, qh, sc in ((0xFF, 0xFF, 127), (0x00, 0x00, 127), (0xFF, 0xFF, 0x80), (0x00, 0x00, 0x80), (0xF0, 0x33, 0x81)):
        b6 = np.zeros((rows * 4, 210), np.uint8)
        b6[:, 0:128] = ql
        b6[:, 128:192] = qh
        b6[:, 192:208] = sc
        b6[:, 208:210] = np.frombuffer(np.float16(0.003).tobytes(), np.uint8)
        got = be.matmul(xe, T, qm(b6.reshape(-1), Q6_K, in_dim, rows))
        assert be.last_kernel() == NAME[Q6_K]
        assert_bits(got, oracle.matmul(Q6_K, b6.reshape(-1), in_dim, rows, xe, T), f"Q6_K ql {ql:#x} qh {qh:#x} sc {sc:#x}")


def test_row_block_kernel_at_the_8b_shapes(be):
    """The four projections of an 8B-shaped layer at verify batches of 4 and 8."""
    for t, in_dim, out_dim in ((Q4_K, 4096, 4096), (Q4_K, 4096, 1024), (Q4_K, 4096, 14336), (Q6_K, 14336, 4096)):
        raw = synth_weights(t, in_dim, out_dim, seed=5)
        w = qm(raw, t, in_dim, out_dim)
        for T in (4, 8):
            x = synth_x(T, in_dim, seed=T)
            got = be.matmul(x, T, w)
            assert be.last_kernel() == NAME[t]
            assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), f"type {t} {in_dim}->{out_dim} at {T} tokens")
        be.evict(w)


def test_default_routing_of_few_token_batches():
    """Without tuning: Q6_K goes to the row-block kernel from four tokens, Q4_K and Q5_K from five, all up to eight;
    one token never, nine and more to the small-batch GEMM.  Shapes the kernel measured slower on stay off it: from
    six tokens Q6_K matrices of more than 4096 rows, Q4_K / Q5_K rows of more than 5120 inputs with more than 4096
    rows.  A batch that the GEMV kernel's LDS cannot hold at once (long rows) goes to the small-batch GEMM however
    few its tokens, instead of reading the weights once per part.  Same bits everywhere."""
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()
    try:
        for t, T, want in ((Q6_K, 1, "ogm_gemv_kernel<FmtQ6K,gemv>"), (Q6_K, 2, "ogm_gemv_kernel<FmtQ6K,gemm>"),
                           (Q6_K, 4, NAME[Q6_K]), (Q6_K, 8, NAME[Q6_K]), (Q6_K, 9, "ogm_gemm_sb_q6k_kernel"),
                           (Q4_K, 4, "ogm_gemv_kernel<FmtQ4K,gemm>"), (Q4_K, 5, NAME[Q4_K]), (Q4_K, 8, NAME[Q4_K]),
                           (Q4_K, 16, "ogm_gemm_sb_q4k_kernel"),
                           (Q5_K, 3, "ogm_gemv_kernel<FmtQ5K,gemm>"), (Q5_K, 8, NAME[Q5_K]), (Q5_K, 9, "ogm_gemm_sb_q5k_kernel")):
            raw = synth_weights(t, 1024, 48, seed=T)
            x = synth_x(T, 1024, seed=T)
            got = b.matmul(x, T, qm(raw, t, 1024, 48))
            assert b.last_kernel() == want, (t, T, b.last_kernel())
            assert_bits(got, oracle.matmul(t, raw, 1024, 48, x, T), f"type {t} at {T} tokens")
        for t, in_dim, out_dim, T, want in (
                (Q6_K, 1024, 4100, 5, NAME[Q6_K]), (Q6_K, 1024, 4100, 7, "ogm_gemm_sb_q6k"),       # many rows: to 5 tokens only
                (Q6_K, 1024, 8200, 4, "ogm_gemv_kernel<FmtQ6K,gemm>"),
                (Q4_K, 8192, 4096, 6, NAME[Q4_K]), (Q4_K, 8192, 4100, 6, "ogm_gemm_sb_q4k"),        # long rows: few rows only
                (Q4_K, 5120, 8200, 5, NAME[Q4_K]), (Q4_K, 5120, 8200, 7, "ogm_gemm_sb_q4k"),
                (Q6_K, 28672, 300, 2, "ogm_gemv_kernel<FmtQ6K,gemm>"), (Q6_K, 28672, 300, 3, "ogm_gemm_sb_q6k"),   # parts of two tokens
                (Q6_K, 53248, 70, 2, "ogm_gemm_sb_q6k"), (Q4_K, 16384, 200, 3, "ogm_gemv_kernel<FmtQ4K,gemm>"),
                (Q4_K, 16384, 200, 4, "ogm_gemm_sb_q4k")):
            raw = synth_weights(t, in_dim, out_dim, seed=T + out_dim)
            x = synth_x(T, in_dim, seed=T)
            w = qm(raw, t, in_dim, out_dim)
            got = b.matmul(x, T, w)
            assert b.last_kernel().startswith(want), (t, in_dim, out_dim, T, b.last_kernel())
            assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), f"type {t} {in_dim}->{out_dim} at {T} tokens")
            b.evict(w)
    finally:
        b.close()

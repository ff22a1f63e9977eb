"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Bar: activation quantization and per-block integer sums bit-exact; f32 outputs
within 1e-3 relative / 1e-5 absolute (they are in fact expected bit-identical, and the tests
report that separately so a regression in the stronger property is visible)."""
import re
import sys

import numpy as np
import pytest

import oracle
from helpers import (BLOCK, FLAT32, IQ4_NL, Q3_K, Q4_0, Q4_K, Q5_0, Q5_K, Q6_K, Q8_0, NextByte, activations, activations_t, cpu_rs_weights,
                     fixture_row, k_fixture, row_bytes, synth_weights, synth_x)
from test_oracle_quantize import adversarial_blocks

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-3, 1e-5  # the stated contract for f32 outputs


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


# The library takes its tiled matrix-core GEMMs from 17 tokens on (below that the GEMV kernel in chunks
# of 8 tokens is faster) and gives batches of up to 64 or 128 tokens of Q4_K, Q5_K and Q6_K to a
# small-batch kernel; these tests run the tiled kernels from 9 tokens on and keep the small-batch
# kernel out, so that tiles with 9, 10, 12 or 16 tokens are covered too.  The small-batch kernel has
# tests of its own, and test_gemm_threshold_default checks the library's own choices.
GEMM_FROM = 9


# Every test of this module runs three times: with the K-quant matrices' prefill planes built on first
# use and kept (gemm_plane_cache_mb > 0) and read by a kernel whose waves all multiply, here whatever the
# grid, from 32 tokens ("planes": ogm_gemm_q*_dma_kernel, 128-row tiles; "planes64": ogm_gemm_q*_dmx_kernel,
# 64-row tiles, the f32 step between the matrix instructions, wherever its types allow), and with none
# ("unpack": the feeding waves unpack the weights on every call).  Same bits every way.
@pytest.fixture(scope="module", params=["planes", "planes64", "unpack"])
def be(request):
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()  # raises if the HIP library or the device is missing: no fallback
    say("device:", b.device_name(), "mode:", request.param)
    b.set_tuning("gemm_min_tokens", GEMM_FROM)
    b.set_tuning("gemm_small_max_tokens", 1)
    b.set_tuning("gemm_medium", 1)   # the medium-batch kernel has tests of its own below
    b.set_tuning("gemv_mma", 0)      # the few-token row-block kernel has tests of its own (test_gpu_few_tokens.py)
    b.set_tuning("gemm_sb_waves", 8)
    b.set_tuning("gemm_plane_cache_mb", 0 if request.param == "unpack" else 65536)
    b.set_tuning("gemm_plane_kernel", 2)
    b.set_tuning("gemm_interleave", 2 if request.param == "planes64" else 1)
    b.plane_mode = request.param
    yield b
    b.close()


class _TiledPlaneKernel(str):
    """Name of the plane kernel that has no 64-row variant: equal to both names of its family."""

    def __eq__(self, other):
        return other in (str(self) + "_kernel", str(self) + "_r64_kernel")

    def __ne__(self, other):
        return not self.__eq__(other)

    def startswith(self, prefix, *a):
        return (str(self) + "_kernel").startswith(prefix, *a) or (str(self) + "_r64_kernel").startswith(prefix, *a)

    __hash__ = str.__hash__


def kname(b):
    """The last kernel's name as the tests of the unpacking kernels expect it: ogm_gemm_q*_dma_kernel as its
    family's tiled kernel (of either row tiling).  Checks that the name fits the mode the backend runs in."""
    name = b.last_kernel()
    mode = getattr(b, "plane_mode", None)   # None: a context with no tuning reads planes on large grids
    m = re.match(r"ogm_gemm_q(6k|3k|4k|5k)_dm([ax])_kernel$", name)
    if m:
        assert mode is None or mode == ("planes64" if m.group(2) == "x" else "planes") or \
            (mode == "planes64" and m.group(1) == "3k"), name   # (Q3_K has no 64-row kernel)
        return _TiledPlaneKernel({"6k": "ogm_gemm_q6k_i8", "3k": "ogm_gemm_q3k_i8", "4k": "ogm_gemm_q4k_i8p",
                                  "5k": "ogm_gemm_q5k_i8p"}[m.group(1)])
    return name


def qm(raw, t, in_dim, out_dim):
    from orangu_amd import QuantMatrix
    return QuantMatrix(np.ascontiguousarray(raw), t, in_dim, out_dim)


def assert_close(got, want, what):
    got = np.asarray(got, np.float32).reshape(-1)
    want = np.asarray(want, np.float32).reshape(-1)
    assert got.shape == want.shape, what
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    tol = RTOL * np.abs(want.astype(np.float64)) + ATOL
    bad = np.nonzero(~(err <= tol))[0]
    assert bad.size == 0, f"{what}: {bad.size} of {got.size} outside 1e-3/1e-5, first {bad[:5]} " \
                          f"got {got[bad[:5]]} want {want[bad[:5]]}"


def assert_bits(got, want, what):
    got = np.asarray(got, np.float32).reshape(-1)
    want = np.asarray(want, np.float32).reshape(-1)
    same = got.view(np.uint32) == want.view(np.uint32)
    assert same.all(), f"{what}: {(~same).sum()} of {got.size} differ in bits; first at " \
                       f"{np.nonzero(~same)[0][:5]} got {got[~same][:5]} want {want[~same][:5]}"


# ---------------------------------------------------------------- formats

def test_f16_scale_conversion_matches_quant_rs_for_all_inputs(be):
    """quant.rs:511-528 / :1671-1690 on the device conversion."""
    bits = np.arange(65536, dtype=np.uint16)
    got = be.f16_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


@pytest.mark.parametrize("t", [Q8_0, Q5_0, Q4_0, IQ4_NL, Q3_K, Q4_K, Q5_K, Q6_K])
def test_upload_download_round_trip(be, t):
    """unrepack(repack(W)) == W through the device."""
    bb, bel = BLOCK[t]
    in_dim, out_dim = bel * 5, 77
    raw = np.random.default_rng(t).integers(0, 256, row_bytes(t, in_dim) * out_dim, dtype=np.uint8)
    w = qm(raw, t, in_dim, out_dim)
    assert np.array_equal(be.download(w), raw)


# ---------------------------------------------------------------- quantizer (bit-exact)

@pytest.mark.parametrize("per_256", [False, True])
def test_quantizer_bit_exact_on_adversarial_and_random_blocks(be, per_256):
    """vecdot.rs:4259-4410 cases plus random data, against the oracle's scalar definition."""
    rng = np.random.default_rng(17)
    tiny = np.full(256, 1e-39, np.float32)  # denormal scale: inv overflows to inf on the CPU
    tiny[3] = -3e-39
    x = np.concatenate([
        np.tile(adversarial_blocks(), 8),                       # 1792
        rng.standard_normal(4096).astype(np.float32) * 3,
        (rng.integers(-254, 255, 2048) * 0.5).astype(np.float32),
        tiny, np.zeros(256, np.float32),
    ])
    x = x[: x.size // 256 * 256]
    fn = oracle.quantize_act_k_row if per_256 else oracle.quantize_act
    wq, wd, ws = fn(x)
    q, d, s = be.quantize_act(x, per_256)
    assert np.array_equal(q, wq), np.nonzero(q != wq)[0][:10]
    assert np.array_equal(d.view(np.uint32), wd.view(np.uint32))
    assert np.array_equal(s, ws)


def test_quantizer_ties_round_away_from_zero(be):
    """vecdot.rs:4395-4410."""
    x = np.full(256, 254.0, np.float32)
    x[1], x[2], x[3], x[4] = 1.0, 3.0, -1.0, -3.0
    for per_256 in (False, True):
        q, d, _ = be.quantize_act(x, per_256)
        assert (q[1], q[2], q[3], q[4]) == (1, 2, -1, -2) and d[0] == 2.0


# ---------------------------------------------------------------- integer stage (bit-exact)

@pytest.mark.parametrize("t,in_dim,out_dim,T", [
    (Q4_K, 256, 5, 1), (Q4_K, 2048, 37, 3), (Q4_K, 4864, 9, 1),
    (Q5_K, 256, 5, 1), (Q5_K, 2048, 37, 3), (Q5_K, 4864, 9, 2),
    (Q3_K, 256, 5, 1), (Q3_K, 2048, 37, 3), (Q3_K, 5632, 9, 2),
    (Q6_K, 256, 5, 1), (Q6_K, 2048, 37, 3), (Q6_K, 4864, 9, 2),
    (Q8_0, 96, 11, 1), (Q8_0, 896, 19, 3), (Q8_0, 4864, 7, 1),
    (Q5_0, 96, 11, 1), (Q5_0, 896, 19, 3), (Q4_0, 32, 5, 2), (Q4_0, 4864, 7, 1), (IQ4_NL, 896, 19, 3), (IQ4_NL, 4864, 7, 2),
])
def test_block_integer_sums_bit_exact(be, t, in_dim, out_dim, T):
    raw = np.concatenate([fixture_row(t, in_dim, 100 + o) for o in range(out_dim)])
    x = np.concatenate([activations_t(in_dim, k) for k in range(T)])
    w = qm(raw, t, in_dim, out_dim)
    isum, imin = be.dump_block_sums(x, T, w)
    wi, wm = oracle.block_sums(t, raw, in_dim, out_dim, x, T)
    assert np.array_equal(isum, wi)
    if t in (Q4_K, Q5_K):
        assert np.array_equal(imin, wm)


# ---------------------------------------------------------------- GEMV / matmul values

CHECK = [(Q8_0, 896), (Q8_0, 4864), (Q4_K, 256), (Q4_K, 4864), (Q6_K, 256), (Q6_K, 4864),
         (Q4_K, 2048), (Q6_K, 5632), (Q5_K, 256), (Q5_K, 3072), (Q5_K, 4864), (Q3_K, 256), (Q3_K, 2048),
         (Q3_K, 5632), (Q5_0, 896), (Q5_0, 4864), (Q4_0, 32), (Q4_0, 896), (Q4_0, 4864), (IQ4_NL, 896), (IQ4_NL, 4864)]


@pytest.mark.parametrize("t,in_dim", CHECK)
@pytest.mark.parametrize("seed", [1, 7, 99])
def test_gemv_matches_cpu_matmul_on_reference_fixtures(be, t, in_dim, seed):
    """The reference's `check` / `k_row` fixtures (vecdot.rs:3436-3526, 4011-4040): matmul at
    n_tokens == 1 against CpuBackend::matmul, and against dequantize . x within the reference's
    own budget."""
    out_dim = 13
    raw = np.concatenate([fixture_row(t, in_dim, seed + 1000 * o) for o in range(out_dim)])
    x = activations(in_dim)
    w = qm(raw, t, in_dim, out_dim)
    got = be.matmul(x, 1, w)
    want = oracle.matmul(t, raw, in_dim, out_dim, x, 1)
    assert_close(got, want, "matmul T=1")
    assert_bits(got, want, "matmul T=1")
    ref = oracle.matmul_dequant(t, raw, in_dim, out_dim, x, 1).reshape(-1)
    rb = row_bytes(t, in_dim)
    for o in range(out_dim):
        wrow = oracle.dequantize(t, raw[o * rb:(o + 1) * rb], in_dim).astype(np.float64)
        mag = np.abs(wrow * x).sum()
        budget = 0.01 if t in FLAT32 else 0.02
        assert abs(float(got[o]) - float(ref[o])) <= budget * max(mag, 1e-6)


@pytest.mark.parametrize("t", [Q8_0, Q5_0, Q4_0, IQ4_NL, Q3_K, Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("T", [1, 2, 5, 8, 13])
def test_matmul_decode_matches_cpu_and_each_token_alone(be, t, T):
    """backend/cpu.rs:623-650: a decode batch's row t is what token t gives alone."""
    in_dim = 128 if t in FLAT32 else 512
    out_dim = 7
    nb = NextByte(0x0051AB1E5EED)
    raw = cpu_rs_weights(t, in_dim, out_dim, nb) if t not in (Q6_K, Q3_K) else np.concatenate(
        [fixture_row(t, in_dim, 5 + o) for o in range(out_dim)])
    x = np.array([np.float32(nb()) / np.float32(255.0) * np.float32(2.0) - np.float32(1.0)
                  for _ in range(T * in_dim)], np.float32)
    w = qm(raw, t, in_dim, out_dim)
    got = be.matmul_decode(x, T, w).reshape(T, out_dim)
    want = oracle.matmul_decode(t, raw, in_dim, out_dim, x, T)
    assert_close(got, want, "matmul_decode")
    assert_bits(got, want, "matmul_decode")
    for k in range(T):
        alone = be.matmul(x[k * in_dim:(k + 1) * in_dim], 1, w)
        assert_bits(got[k], alone, f"token {k} alone")


@pytest.mark.parametrize("t", [Q8_0, Q5_0, Q4_0, IQ4_NL, Q3_K, Q4_K, Q5_K, Q6_K])
def test_matmul_multi_token_matches_cpu_gemm(be, t):
    """backend/cpu.rs:544-582 shapes: in = 3 blocks, out = 11 (odd), T in 1,2,5,77,3,1 from one
    reused backend; matmul at T > 1 follows the CPU GEMM kernels."""
    in_dim = BLOCK[t][1] * 3
    out_dim = 11
    raw = cpu_rs_weights(t, in_dim, out_dim, NextByte(0x9E3779B97F4A7C15)) if t not in (Q6_K, Q3_K) else \
        np.concatenate([fixture_row(t, in_dim, 50 + o) for o in range(out_dim)])
    w = qm(raw, t, in_dim, out_dim)
    for T in (1, 2, 5, 77, 3, 1):
        i = np.arange(T * in_dim)
        x = ((i % 29).astype(np.float32) - np.float32(14.0)) * np.float32(0.037)
        got = be.matmul(x, T, w)
        want = oracle.matmul(t, raw, in_dim, out_dim, x, T)
        assert got.size == T * out_dim
        assert_close(got, want, f"matmul T={T}")
        assert_bits(got, want, f"matmul T={T}")


@pytest.mark.parametrize("t", [Q3_K, Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("in_dim", [256, 2048, 8192])
def test_k_gemm_fixture(be, t, in_dim):
    """vecdot.rs:4479-4513: 5 rows x 7 tokens, seed 4242."""
    raw, x = k_fixture(t, in_dim, 5, 7, 4242)
    got = be.matmul(x, 7, qm(raw, t, in_dim, 5)).reshape(7, 5)
    want = oracle.k_gemm_t(t, raw, in_dim, 5, x, 7).T
    assert_close(got, want, "k_gemm")
    assert_bits(got, want, "k_gemm")


@pytest.mark.parametrize("t", [Q3_K, Q4_K, Q5_K, Q6_K])
def test_gemm_result_is_independent_of_the_batch_size(be, t):
    """vecdot.rs:4522-4549: exact equality."""
    in_dim, out_dim = 512, 4
    raw, x = k_fixture(t, in_dim, out_dim, 8, 77)
    w = qm(raw, t, in_dim, out_dim)
    full = be.matmul(x, 8, w).reshape(8, out_dim)
    for n in (2, 3, 5, 7):
        part = be.matmul(x[: n * in_dim], n, w).reshape(n, out_dim)
        assert_bits(part, full[:n], f"{n} of 8")


def test_matmul_batch_equals_single_calls_and_stripes(be):
    """Backend::matmul_batch (mod.rs:362-366) with token stripes (mod.rs:154-172)."""
    from orangu_amd import MatmulOp
    in_dim = 512
    ws = [qm(np.concatenate([fixture_row(t, in_dim, 9 + o) for o in range(od)]), t, in_dim, od)
          for t, od in ((Q4_K, 6), (Q6_K, 9), (Q8_0, 5))]
    ops = []
    for k, (w, T) in enumerate(zip(ws, (1, 4, 11))):
        ops.append(MatmulOp(np.concatenate([activations_t(in_dim, k + j) for j in range(T)]), T, w))
    outs = be.matmul_batch(ops, max_tokens_per_phase=3)
    for op, y in zip(ops, outs):
        assert_bits(y, be.matmul(op.x, op.n_tokens, op.w) if op.n_tokens <= 3 else
                    np.concatenate([be.matmul(op.x[s * in_dim:min(op.n_tokens, s + 3) * in_dim],
                                              min(op.n_tokens, s + 3) - s, op.w)
                                    for s in range(0, op.n_tokens, 3)]), "stripe")
    outs = be.matmul_batch_decode(ops)
    for op, y in zip(ops, outs):
        assert_bits(y, be.matmul_decode(op.x, op.n_tokens, op.w), "decode batch")


def test_matmul_batch_with_an_op_without_tokens_in_front(be):
    """An op with n_tokens == 0 brings no input and must not stand in for the input of the op
    behind it (both would otherwise sit at the same staging offset)."""
    from orangu_amd import MatmulOp
    in_dim = 512
    w = qm(np.concatenate([fixture_row(Q4_K, in_dim, 3 + o) for o in range(7)]), Q4_K, in_dim, 7)
    w6 = qm(np.concatenate([fixture_row(Q6_K, in_dim, 5 + o) for o in range(4)]), Q6_K, in_dim, 4)
    xa, xb = activations_t(in_dim, 1), np.concatenate([activations_t(in_dim, 2 + j) for j in range(3)])
    empty = np.zeros(0, np.float32)
    for ops in ([MatmulOp(empty, 0, w), MatmulOp(xa, 1, w), MatmulOp(xb, 3, w6)],
                [MatmulOp(xa, 1, w), MatmulOp(empty, 0, w6), MatmulOp(xb, 3, w6), MatmulOp(empty, 0, w)],
                [MatmulOp(empty, 0, w), MatmulOp(empty, 0, w6)]):
        for decode in (False, True):
            outs = (be.matmul_batch_decode if decode else be.matmul_batch)(ops)
            for op, y in zip(ops, outs):
                assert np.asarray(y).size == op.n_tokens * op.w.out_dim
                if op.n_tokens:
                    want = (oracle.matmul_decode if decode else oracle.matmul)(
                        op.w.ggml_type(), op.w.raw_bytes(), in_dim, op.w.out_dim, op.x, op.n_tokens)
                    assert_bits(y, want, "batch with an empty op")


@pytest.mark.parametrize("T", [2, 5, 9])
@pytest.mark.parametrize("in_dim", [256, 1024, 4096])
def test_multi_token_quantizer_matches_act_q8k_and_act_q8flat(be, T, in_dim):
    """The quantizer as the multi-token matmuls launch it, against ActQ8K::quantize and
    ActQ8Flat::quantize (vecdot.rs:1858-1910, 2483-2525): int8 values, scales and the per-32 sums bit
    for bit (the reference's 4-token interleave undone on the host), and the f16 pairs
    (floor(bsum / 64), bsum mod 64) the K-quant GEMMs' first pass reads."""
    x = synth_x(T, in_dim, seed=40 + T).reshape(T, in_dim)
    x[0, :32] = 0.0                       # an all-zero block: scale 0
    x[T - 1, 5] = np.float32("nan")       # NaN quantizes to 0 and does not enter the maximum
    x[T - 1, 40] = 3.0e38
    # per 256
    q, d, sums, bsum, bs16 = be.quantize_act_tokens(x, in_dim, T, True)
    wq, wd, wb = oracle.act_q8k_quantize(x, in_dim, T)     # [tile][in/32][4][32], [tile][in/256][4], [tile][in/256][4][8]
    for t in range(T):
        tl, k = divmod(t, 4)
        assert np.array_equal(q[t], wq[tl, :, k, :].reshape(-1)), f"token {t}: q"
        assert np.array_equal(d[t].view(np.uint32), wd[tl, :, k].view(np.uint32)), f"token {t}: d"
        assert np.array_equal(bsum[t], wb[tl, :, k, :].reshape(-1)), f"token {t}: bsum"
        rq, rd, rs = oracle.quantize_act_k_row(x[t])      # the decode quantizer gives the same values
        assert np.array_equal(q[t], rq) and np.array_equal(sums[t], rs)
        b = bsum[t].astype(np.int32).reshape(-1, 8)
        h = bs16[t].view(np.float16).astype(np.float64).reshape(-1, 16)
        assert np.array_equal(h[:, :8], b >> 6) and np.array_equal(h[:, 8:], b & 63), f"token {t}: bs16"
    # per 32
    q, d, sums, bsum, _ = be.quantize_act_tokens(x, in_dim, T, False)
    wq, wd = oracle.act_q8flat_quantize(x, in_dim, T)      # [tile][in/32][4][32], [tile][in/32][4]
    for t in range(T):
        tl, k = divmod(t, 4)
        assert np.array_equal(q[t], wq[tl, :, k, :].reshape(-1)), f"token {t}: q (per 32)"
        assert np.array_equal(d[t].view(np.uint32), wd[tl, :, k].view(np.uint32)), f"token {t}: d (per 32)"
        assert np.array_equal(bsum[t], q[t].astype(np.int32).reshape(-1, 32).sum(axis=1))
        assert np.array_equal(sums[t], q[t].astype(np.int32).reshape(-1, 16).sum(axis=1))


def test_row_views_share_bytes_but_not_handles(be):
    """QuantMatrix::rows (loader.rs:627-646): a view's cache key differs from its parent's."""
    in_dim, out_dim = 512, 12
    raw = np.concatenate([fixture_row(Q4_K, in_dim, 3 + o) for o in range(out_dim)])
    w = qm(raw, Q4_K, in_dim, out_dim)
    x = activations(in_dim)
    full = be.matmul(x, 1, w)
    part = be.matmul(x, 1, w.rows(4, 5))
    assert_bits(part, full[4:9], "rows view")
    assert be.upload(w) == be.upload(w) and be.upload(w) != be.upload(w.rows(4, 5))


def test_error_statuses(be):
    from orangu_amd import OgmError, QuantMatrix
    with pytest.raises(ValueError):
        QuantMatrix(np.zeros(144, np.uint8), Q4_K, 128, 1)
    w = qm(fixture_row(Q4_K, 256, 1), Q4_K, 256, 1)
    with pytest.raises(ValueError):
        be.matmul(np.zeros(100, np.float32), 1, w)
    with pytest.raises(OgmError):
        be.set_tuning("no_such_key", 1)
    assert be.matmul(np.zeros(0, np.float32), 0, w).size == 0


# ---------------------------------------------------------------- benchmark shapes

@pytest.mark.parametrize("t,in_dim,out_dim", [
    (Q8_0, 4096, 4096),     # config 1
    (Q4_K, 4096, 14336),    # config 2 gate/up
    (Q4_K, 14336, 4096),    # config 2 down
    (Q4_K, 4096, 1024),     # config 3 k/v
    (Q6_K, 14336, 4096),    # config 5 ffn_down
    (Q5_K, 4096, 4096), (Q5_K, 14336, 4096),   # the same shapes in Q5_K
    (Q3_K, 4096, 4096), (Q3_K, 14336, 4096),   # and in Q3_K
    (Q4_0, 4096, 4096), (Q5_0, 14336, 4096), (IQ4_NL, 4096, 14336),
])
def test_benchmark_shapes_match_cpu(be, t, in_dim, out_dim):
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim)
    x = synth_x(1, in_dim, seed=3)
    w = qm(raw, t, in_dim, out_dim)
    say("shape", t, in_dim, out_dim)
    got = be.matmul(x, 1, w)
    want = oracle.matmul(t, raw, in_dim, out_dim, x, 1)
    assert_close(got, want, "full-size GEMV")
    assert_bits(got, want, "full-size GEMV")
    for waves in (1, 2, 3, 16):
        be.set_tuning("gemv_wg_waves", waves)
        assert_bits(be.matmul(x, 1, w), want, f"wg_waves={waves}")
    be.set_tuning("gemv_wg_waves", 0)


@pytest.mark.parametrize("out_dim", [4096, 1024])
@pytest.mark.parametrize("T", [4, 8])
def test_q4k_attention_projections_at_verify_batches(be, out_dim, T):
    """Config 3: the Q4_K attention projections 4096 -> 4096 (q / o) and 4096 -> 1024 (k / v) at the
    speculative-verify batches 4 and 8, full size, through Backend::matmul (GEMM float order) and
    Backend::matmul_decode (each row the single-token kernel): bit for bit."""
    in_dim = 4096
    raw = synth_weights(Q4_K, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T)
    w = qm(raw, Q4_K, in_dim, out_dim)
    say("verify batch", out_dim, T)
    got = be.matmul(x, T, w)
    want = oracle.matmul(Q4_K, raw, in_dim, out_dim, x, T)
    assert_close(got, want, "matmul")
    assert_bits(got, want, "matmul")
    got = be.matmul_decode(x, T, w)
    want = oracle.matmul_decode(Q4_K, raw, in_dim, out_dim, x, T)
    assert_close(got, want, "matmul_decode")
    assert_bits(got, want, "matmul_decode")
    one = be.matmul(x.reshape(T, in_dim)[T - 1], 1, w)
    assert_bits(np.asarray(got).reshape(T, out_dim)[T - 1], one, "matmul_decode row == the token alone")


@pytest.mark.parametrize("M", [128, 512, 2048])
def test_prefill_gemm_at_the_benchmark_sizes(be, M):
    """Config 4: Q4_K 4096 -> 14336 over M = 128 / 512 / 2048 tokens at full size with the library's
    own kernel choice, against the CPU GEMM on sampled rows (the first, a middle and the last row
    tile) bit for bit, and -- the size-independent property over every row -- batch independence:
    the first 16 token rows of the result equal the matmul of those 16 tokens alone
    (vecdot.rs:4522-4549)."""
    in_dim, out_dim = 4096, 14336
    raw = synth_weights(Q4_K, in_dim, out_dim, seed=77)
    x = synth_x(M, in_dim, seed=M)
    w = qm(raw, Q4_K, in_dim, out_dim)
    be.set_tuning("gemm_min_tokens", 0)
    be.set_tuning("gemm_small_max_tokens", 0)
    be.set_tuning("gemm_sb_waves", 0)
    try:
        got = np.asarray(be.matmul(x, M, w)).reshape(M, out_dim)
        say("prefill GEMM", M, be.last_kernel())
        head = np.asarray(be.matmul(x.reshape(M, in_dim)[:16], 16, w)).reshape(16, out_dim)
    finally:
        be.set_tuning("gemm_min_tokens", GEMM_FROM)
        be.set_tuning("gemm_small_max_tokens", 1)
        be.set_tuning("gemm_sb_waves", 8)
    rows = np.r_[0:32, 7000:7032, out_dim - 32:out_dim]
    rb = row_bytes(Q4_K, in_dim)
    sub = np.concatenate([raw[r * rb:(r + 1) * rb] for r in rows])
    want = oracle.matmul(Q4_K, sub, in_dim, rows.size, x, M).reshape(M, rows.size)
    assert_close(got[:, rows], want, "sampled rows")
    assert_bits(got[:, rows], want, "sampled rows")
    assert_bits(got[:16], head, "batch independence over all rows")


def test_argmax_follows_total_cmp(be):
    """sampling::argmax (sampling.rs:336-343): max_by over total_cmp -- the last of equal maxima,
    -0 below +0, a positive NaN above every number, a negative NaN below."""
    from oracle import llama_ref as R
    nan, inf = np.float32("nan"), np.float32("inf")
    neg_nan = np.array([0xFFC00000], np.uint32).view(np.float32)[0]
    cases = [[1.0, 5.0, 2.0, 5.0, 0.0], [-3.0], [-0.0, 0.0, -0.0], [0.0, -0.0], [1.0, nan, 7.0], [neg_nan, -inf, neg_nan],
             [-inf, -inf], [inf, 3.0, inf, nan, nan], [neg_nan], [neg_nan, neg_nan]]
    rng = np.random.default_rng(12)
    big = rng.standard_normal(128256).astype(np.float32)
    big[[5, 70000, 128255]] = big.max() + 1.0
    cases += [big, np.where(rng.random(70001) < 0.01, nan, rng.standard_normal(70001)).astype(np.float32),
              np.zeros(513, np.float32), -np.zeros(1000, np.float32)]
    for c in cases:
        c = np.asarray(c, np.float32)
        assert be.argmax(c) == R.argmax(c), c[:8]


def test_q6k_vocab_projection_batches_1_4_8(be):
    """Config 3: Q6_K 4096 -> 128256 at batch 1, 4, 8 (rows sampled against the oracle; linearity
    in x as the size-independent property over all rows)."""
    in_dim, out_dim = 4096, 128256
    raw = synth_weights(Q6_K, in_dim, out_dim, seed=6)
    w = qm(raw, Q6_K, in_dim, out_dim)
    x = synth_x(8, in_dim, seed=8)
    say("q6k vocab upload+matmul")
    rows = np.r_[0:64, 64000:64064, out_dim - 64:out_dim]
    rb = row_bytes(Q6_K, in_dim)
    sub = np.concatenate([raw[r * rb:(r + 1) * rb] for r in rows])
    for T in (1, 4, 8):
        got = be.matmul_decode(x[:T], T, w).reshape(T, out_dim)
        want = oracle.matmul_decode(Q6_K, sub, in_dim, rows.size, x[:T], T)
        assert_bits(got[:, rows], want, f"decode T={T}")
        got = be.matmul(x[:T], T, w).reshape(T, out_dim)
        want = oracle.matmul(Q6_K, sub, in_dim, rows.size, x[:T], T)
        assert_bits(got[:, rows], want, f"matmul T={T}")
    # all rows: power-of-two scaling of x scales y exactly (quantizer scale follows, ints equal)
    y1 = be.matmul(x[:1], 1, w)
    y2 = be.matmul(x[:1] * np.float32(4.0), 1, w)
    assert_bits(y2, y1 * np.float32(4.0), "scaling by 4")


# ---------------------------------------------------------------- prefill GEMM on MFMA

def plane_kernel(base, T, outs):
    """Name of the int8 plane kernel a K-quant GEMM launch takes: `base` (e.g. "ogm_gemm_q4k_i8p") on
    128-row tiles, or its 64-row variant when those tiles still come one to a compute unit."""
    outs = outs if isinstance(outs, (tuple, list)) else (outs,)
    small = ((T + 127) // 128) * sum((o + 63) // 64 for o in outs) <= 256
    return base + ("_r64_kernel" if small else "_kernel")


def tile_rows(be, rows):
    """gemm_tile_rows: 64 makes the feeding-wave kernels take their 64-row tiles whatever the grid, 0 the default."""
    be.set_tuning("gemm_tile_rows", rows)


@pytest.mark.parametrize("in_dim,out_dim,T", [
    (1024, 64, 9), (1024, 100, 64), (2048, 37, 128), (4096, 200, 130), (1024, 16, 300), (8192, 70, 33),
    (256, 5, 9), (512, 130, 17), (768, 64, 129), (1280, 257, 40), (14336, 96, 257), (4096, 1000, 512),
    (256, 5, 257), (2304, 130, 600), (4096, 257, 1030), (1024, 129, 256), (512, 64, 513),
])
def test_mfma_gemm_q4k_matches_cpu_gemm(be, in_dim, out_dim, T):
    """ogm_matmul at n_tokens >= 9 takes the matrix-core kernels; values must equal CpuBackend's
    K-quant GEMM (vecdot.rs:2213-2303): integer sums exact, f32 order the reference's, on both tile
    heights of the int8 plane kernel."""
    raw = synth_weights(Q4_K, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T)
    w = qm(raw, Q4_K, in_dim, out_dim)
    say("gemm", in_dim, out_dim, T)
    want = oracle.matmul(Q4_K, raw, in_dim, out_dim, x, T)
    got = be.matmul(x, T, w)
    assert kname(be) == plane_kernel("ogm_gemm_q4k_i8p", T, out_dim)
    assert_close(got, want, "int8 plane gemm")
    assert_bits(got, want, "int8 plane gemm")
    tile_rows(be, 64)   # the 64-row tiles whatever the grid
    try:
        got = be.matmul(x, T, w)
        assert kname(be) == "ogm_gemm_q4k_i8p_r64_kernel"
        assert_bits(got, want, "int8 plane gemm, 64-row tiles")
    finally:
        tile_rows(be, 0)


@pytest.mark.parametrize("t,in_dim,out_dim,T", [
    (Q4_K, 256, 5, 9), (Q4_K, 1024, 200, 70), (Q4_K, 4096, 96, 128), (Q4_K, 512, 33, 129), (Q5_K, 1024, 130, 140),
    (Q4_K, 2048, 64, 40), (Q5_K, 768, 257, 300), (Q4_K, 14336, 70, 257), (Q4_K, 8192, 100, 100), (Q5_K, 4096, 31, 128),
])
def test_medium_batch_kernel_matches_cpu_gemm(be, t, in_dim, out_dim, T):
    """32 rows x 128 tokens per workgroup, its four waves on different super-blocks, the terms added in order
    (gemm_k_q4_k, vecdot.rs:2213-2303): every bit of the CPU GEMM at ragged rows and tokens, with the operand
    chunks written by the quantizer (from 32 tokens) or by the relayout kernel (below)."""
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T)
    be.set_tuning("gemm_medium", 2)
    try:
        got = be.matmul(x, T, qm(raw, t, in_dim, out_dim))
    finally:
        be.set_tuning("gemm_medium", 1)
    assert be.last_kernel() == ("ogm_gemm_sbw_q4k_kernel" if t == Q4_K else "ogm_gemm_sbw_q5k_kernel")
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), "medium-batch gemm")


def test_medium_batch_kernel_over_several_matrices_and_extreme_ranges(be):
    """q / k / v in one launch (row tiles run through the matrices in turn), and the largest magnitudes the
    integer stage can see: nibbles 15, scales and mins 63, activations +-127."""
    from orangu_amd.hiprt import DeviceBuffer, device_synchronize
    in_dim, T, outs = 1024, 150, (300, 130, 64)
    raws = [synth_weights(Q4_K, in_dim, od, seed=90 + i) for i, od in enumerate(outs)]
    hs = [be.upload_raw(r, Q4_K, in_dim, od) for r, od in zip(raws, outs)]
    x = synth_x(T, in_dim, seed=17)
    xd = DeviceBuffer.from_numpy(x)
    yds = [DeviceBuffer(4 * T * od) for od in outs]
    be.set_tuning("gemm_medium", 2)
    try:
        be.matmul_multi_dev(hs, xd.ptr, T, [y.ptr for y in yds])
        device_synchronize()
        assert be.last_kernel() == "ogm_gemm_sbw_q4k_kernel"
        for r, od, yd in zip(raws, outs, yds):
            assert_bits(yd.to_numpy(np.float32, T * od), oracle.matmul(Q4_K, r, in_dim, od, x, T), f"{od} rows of {outs}")
        blocks = np.zeros((32 * 4, 144), np.uint8)
        blocks[:, 0:2] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
        blocks[:, 2:4] = np.frombuffer(np.float16(0.02).tobytes(), np.uint8)
        blocks[:, 4:16] = 0xFF
        blocks[:, 16:] = 0xFF
        xe = np.full((100, 1024), 127.0, np.float32)
        xe[1::2] *= -1
        xe[:, ::7] = 126.0
        got = be.matmul(xe, 100, qm(blocks.reshape(-1), Q4_K, 1024, 32))
        assert be.last_kernel() == "ogm_gemm_sbw_q4k_kernel"
        assert_bits(got, oracle.matmul(Q4_K, blocks.reshape(-1), 1024, 32, xe, 100), "extreme ranges")
    finally:
        be.set_tuning("gemm_medium", 1)
        for h in hs:
            be.free_weight(h)
        for b in [xd] + yds:
            b.free()


def test_gemm_threshold_default():
    """A context of its own with no tuning.  Q8_0: 8 tokens go through the GEMV kernel in the GEMM's
    float order, 9 through the per-32 types' small-batch GEMM (rows so long that the GEMV kernel would read the
    weights once per part of the batch: from the first token it cannot hold), a launch of many workgroups through
    their tiled GEMM.  Q4_K: 4 tokens through the GEMV kernel, 5 to 8 through the
    row-block kernel, then the small-batch kernel: to 512 tokens over a matrix of up to 2048 rows, to 256 over one
    of up to 4096, to 128 over one of up to 8192, where the medium-batch kernel has the second token tile and a tiled
    kernel what follows; a matrix of many rows leaves the small-batch kernel after 64 tokens, and one of so
    many that 128 x 128 tiles outnumber the compute units has its planes built and read by the kernel whose
    waves all multiply, while a single nearly full token tile over at most 16384 rows goes to the medium-batch kernel.
    Q6_K goes to the 64-row plane kernel wherever that has 128 workgroups and a last token tile more than three
    quarters full, or three token tiles, or 160 workgroups and more than 96 tokens, before the small-batch kernel is
    asked.
    Same bits everywhere."""
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()
    try:
        raw = synth_weights(Q8_0, 1024, 70, seed=3)
        x = synth_x(257, 1024, seed=4)
        w = qm(raw, Q8_0, 1024, 70)
        want = oracle.matmul(Q8_0, raw, 1024, 70, x[:17], 17).reshape(17, 70)
        y8 = b.matmul(x[:8], 8, w)
        assert kname(b).startswith("ogm_gemv_kernel")
        y9 = b.matmul(x[:9], 9, w)
        assert kname(b) == "ogm_gemm_sb_flat_kernel"
        y17 = b.matmul(x[:17], 17, w)
        assert kname(b) == "ogm_gemm_sb_flat_kernel"
        assert_bits(y17, want, "Q8_0, 17 tokens")
        assert_bits(y9, want[:9], "Q8_0, 9 tokens")
        assert_bits(y8, want[:8], "Q8_0, 8 tokens")
        rawl = synth_weights(Q8_0, 14336, 40, seed=23)   # rows of which the GEMV kernel's LDS holds one token's worth
        xl = synth_x(5, 14336, seed=24)
        y = b.matmul(xl[:1], 1, qm(rawl, Q8_0, 14336, 40))
        assert kname(b).startswith("ogm_gemv_kernel")
        y = b.matmul(xl[:2], 2, qm(rawl, Q8_0, 14336, 40))
        assert kname(b) == "ogm_gemm_sb_flat_w16_kernel"
        assert_bits(y, oracle.matmul(Q8_0, rawl, 14336, 40, xl[:2], 2), "Q8_0 of 14336 inputs, 2 tokens")
        y = b.matmul(xl, 5, qm(rawl, Q8_0, 14336, 40))
        assert kname(b) == "ogm_gemm_sb_flat_w16_kernel"   # (few workgroups, rows of many blocks: sixteen waves)
        assert_bits(y, oracle.matmul(Q8_0, rawl, 14336, 40, xl, 5), "Q8_0 of 14336 inputs, 5 tokens")
        rawf = synth_weights(Q8_0, 256, 8300, seed=22)   # 260 row blocks of 32 x 10 token blocks: the tiled kernel
        xf = np.ascontiguousarray(x[:, :256])
        y = b.matmul(xf, 257, qm(rawf, Q8_0, 256, 8300))
        assert kname(b) == "ogm_gemm_flat_kernel"
        assert_bits(y, oracle.matmul(Q8_0, rawf, 256, 8300, xf, 257), "Q8_0, 257 tokens x 8300 rows")
        raw = synth_weights(Q4_K, 1024, 70, seed=5)
        w = qm(raw, Q4_K, 1024, 70)
        want = oracle.matmul(Q4_K, raw, 1024, 70, x, 257).reshape(257, 70)
        # (up to 32 tiles of 64 rows the small-batch kernel keeps batches of up to 512 tokens)
        for n, kernel in ((4, "ogm_gemv_kernel"), (5, "ogm_gemm_fk_kernel<Q4_K>"), (8, "ogm_gemm_fk_kernel<Q4_K>"),
                          (9, "ogm_gemm_sb_q4k_kernel"), (128, "ogm_gemm_sb_q4k_kernel"),
                          (257, "ogm_gemm_sb_q4k_kernel")):
            y = b.matmul(x[:n], n, w)
            assert kname(b).startswith(kernel), (n, kname(b))
            assert_bits(y, want[:n], f"Q4_K, {n} tokens")
        # (up to 64 tiles, up to 256 tokens; three token tiles over so few rows are too few workgroups for the planes)
        raw = synth_weights(Q4_K, 256, 2100, seed=25)
        w = qm(raw, Q4_K, 256, 2100)
        x2 = np.ascontiguousarray(x[:, :256])
        want = oracle.matmul(Q4_K, raw, 256, 2100, x2, 257).reshape(257, 2100)
        for n, kernel in ((160, "ogm_gemm_sb_q4k_kernel"), (256, "ogm_gemm_sb_q4k_kernel"),
                          (257, "ogm_gemm_q4k_i8p_r64_kernel")):
            y = b.matmul(x2[:n], n, w)
            assert kname(b).startswith(kernel), (n, kname(b))
            assert_bits(y, want[:n], f"Q4_K of 2100 rows, {n} tokens")
        # (up to 128 tiles, up to 128 tokens; then the medium-batch kernel has the second token tile, full or not,
        # and the 64-row plane kernel the third)
        raw = synth_weights(Q4_K, 256, 4200, seed=26)
        w = qm(raw, Q4_K, 256, 4200)
        want = oracle.matmul(Q4_K, raw, 256, 4200, x2, 257).reshape(257, 4200)
        for n, kernel in ((128, "ogm_gemm_sb_q4k_kernel"), (129, "ogm_gemm_sbw_q4k_kernel"),
                          (256, "ogm_gemm_sbw_q4k_kernel"), (257, "ogm_gemm_q4k_dmx_kernel")):
            y = b.matmul(x2[:n], n, w)
            assert b.last_kernel() == kernel, (n, b.last_kernel())
            assert_bits(y, want[:n], f"Q4_K of 4200 rows, {n} tokens")
        raw = synth_weights(Q4_K, 768, 70, seed=15)    # three super-blocks a row: tiles of 64 rows, one block wide
        w3 = qm(raw, Q4_K, 768, 70)
        x3 = np.ascontiguousarray(x[:9, :768])
        for n, kernel in ((4, "ogm_gemv_kernel"), (6, "ogm_gemm_fk_kernel<Q4_K>"), (9, "ogm_gemm_sb_q4k_kernel")):
            y = b.matmul(x3[:n], n, w3)
            assert kname(b).startswith(kernel), (n, kname(b))
            assert_bits(y, oracle.matmul(Q4_K, raw, 768, 70, x3[:n], n), f"Q4_K of 768 inputs, {n} tokens")
        raw = synth_weights(Q5_K, 4096, 70, seed=7)    # few workgroups, sixteen super-blocks: sixteen waves
        x4 = synth_x(12, 4096, seed=8)
        y = b.matmul(x4, 12, qm(raw, Q5_K, 4096, 70))
        assert kname(b) == "ogm_gemm_sb_q5k_w16_kernel"
        assert_bits(y, oracle.matmul(Q5_K, raw, 4096, 70, x4, 12), "Q5_K, 12 tokens")
        raw = synth_weights(Q6_K, 256, 8300, seed=6)   # 130 tiles of 64 rows
        w = qm(raw, Q6_K, 256, 8300)
        want = oracle.matmul(Q6_K, raw, 256, 8300, np.ascontiguousarray(x[:97, :256]), 97).reshape(97, 8300)
        # (a token tile of the 64-row plane kernel wants more than 96 tokens; Q6_K takes it from 128 workgroups)
        for n, kernel in ((64, "ogm_gemm_sb_q6k_kernel"), (65, "ogm_gemm_q6k_i8_r64_kernel"), (97, "ogm_gemm_q6k_dmx_kernel")):
            y = b.matmul(np.ascontiguousarray(x[:n, :256]), n, w)
            assert b.last_kernel() == kernel, (n, b.last_kernel())
            assert_bits(y, want[:n], f"Q6_K, {n} tokens")
        raw6 = synth_weights(Q6_K, 512, 3100, seed=16)  # 49 tiles of 64 rows: small batches to 256 tokens; a third
        w6 = qm(raw6, Q6_K, 512, 3100)                   # token tile makes 147 workgroups for the plane kernel
        x6 = np.ascontiguousarray(x[:257, :512])
        want = oracle.matmul(Q6_K, raw6, 512, 3100, x6, 257).reshape(257, 3100)
        for n, kernel in ((128, "ogm_gemm_sb_q6k_kernel"), (192, "ogm_gemm_sb_q6k_kernel"), (256, "ogm_gemm_sb_q6k_kernel"),
                          (257, "ogm_gemm_q6k_dmx_kernel")):
            y = b.matmul(x6[:n], n, w6)
            assert b.last_kernel() == kernel, (n, b.last_kernel())
            assert_bits(y, want[:n], f"Q6_K of 3100 rows, {n} tokens")
        raw = synth_weights(Q4_K, 256, 16600, seed=9)   # 130 tiles of 128 rows x 2 of 128 tokens
        w = qm(raw, Q4_K, 256, 16600)
        x5 = np.ascontiguousarray(x[:129, :256])
        y = b.matmul(x5, 129, w)
        assert b.last_kernel() == "ogm_gemm_q4k_dma_kernel"
        assert_bits(y, oracle.matmul(Q4_K, raw, 256, 16600, x5, 129), "Q4_K, 129 tokens x 16600 rows")
        raw7 = synth_weights(Q4_K, 256, 4000, seed=12)   # 63 tiles of 64 rows x 3 of 128 tokens: the 64-row plane kernel
        x7 = synth_x(300, 256, seed=13)
        y = b.matmul(x7, 300, qm(raw7, Q4_K, 256, 4000))
        assert b.last_kernel() == "ogm_gemm_q4k_dmx_kernel"
        assert_bits(y, oracle.matmul(Q4_K, raw7, 256, 4000, x7, 300), "Q4_K, 300 tokens x 4000 rows")
        y = b.matmul(x5[:128], 128, w)                   # one full token tile, but more 32-row workgroups than one round
        assert b.last_kernel() == "ogm_gemm_q4k_i8p_kernel"
        assert_bits(y, oracle.matmul(Q4_K, raw, 256, 16600, x5[:128], 128), "Q4_K, 128 tokens x 16600 rows")
        y = b.matmul(x5[:90], 90, w)                     # a token tile a third empty: 130 workgroups of 128 rows
        assert b.last_kernel() == "ogm_gemm_q4k_i8p_kernel"
        raw = synth_weights(Q4_K, 256, 16000, seed=10)  # 500 workgroups of 32 rows: the medium-batch kernel's one round
        w = qm(raw, Q4_K, 256, 16000)
        y = b.matmul(x5[:128], 128, w)
        assert b.last_kernel() == "ogm_gemm_sbw_q4k_kernel"
        assert_bits(y, oracle.matmul(Q4_K, raw, 256, 16000, x5[:128], 128), "Q4_K, 128 tokens x 16000 rows")
    finally:
        b.close()


@pytest.mark.parametrize("t", [Q3_K, Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("in_dim,out_dim,T", [
    (256, 5, 9), (1024, 100, 17), (768, 64, 32), (1280, 257, 40), (2048, 37, 64), (14336, 96, 33), (1792, 33, 10),
    (4096, 300, 20), (512, 31, 63), (2304, 130, 100), (1024, 70, 128), (256, 1, 1000),
])
@pytest.mark.parametrize("waves", [8, 16])
def test_small_batch_gemm_matches_cpu_gemm(be, t, in_dim, out_dim, T, waves):
    """The small-batch kernel of the K-quants (a workgroup's eight or sixteen waves on different super-blocks of
    32 rows x 32 tokens, terms added in ascending order afterwards): every bit of gemm_k_q4_k /
    gemm_k_q6_k (vecdot.rs:2213-2303, 2352-2398; Q3_K through gemm_k_q6_k's loop, :2014-2021), at any token count
    it is asked for."""
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T + 2)
    be.set_tuning("gemm_small_max_tokens", 1024)
    be.set_tuning("gemm_sb_waves", waves)
    try:
        got = be.matmul(x, T, qm(raw, t, in_dim, out_dim))
    finally:
        be.set_tuning("gemm_small_max_tokens", 1)
        be.set_tuning("gemm_sb_waves", 8)
    assert kname(be) == {Q3_K: "ogm_gemm_sb_q3k", Q4_K: "ogm_gemm_sb_q4k", Q5_K: "ogm_gemm_sb_q5k", Q6_K: "ogm_gemm_sb_q6k"}[t] + \
        ("_w16_kernel" if waves == 16 else "_kernel")
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), "small-batch gemm")


@pytest.mark.parametrize("t,block,hi", [(Q4_K, 144, 0xFF), (Q5_K, 176, 0xFF), (Q6_K, 210, 0x7F), (Q6_K, 210, 0x80),
                                        (Q3_K, 110, 0xFF), (Q3_K, 110, 0x00)])
@pytest.mark.parametrize("waves", [8, 16])
def test_small_batch_gemm_extreme_integer_ranges(be, t, block, hi, waves):
    """Every weight bit and scale byte at its extreme (Q6_K: scales +127 and -128), activations +-127."""
    in_dim, out_dim, T = 1024, 40, 24
    blocks = np.full((out_dim * 4, block), 0xFF, np.uint8)
    if t == Q6_K:
        blocks[:, 192:208] = hi
        blocks[:, 208:210] = np.frombuffer(np.float16(0.003).tobytes(), np.uint8)
    elif t == Q3_K:   # hmask[32] | qs[64] | scales[12] | d: scales 63 - 32 = 31 or 0 - 32 = -32, weights 3 or (hmask 0) -1
        blocks[:, 96:108] = hi
        blocks[1::2, 0:32] = 0x00
        blocks[:, 108:110] = np.frombuffer(np.float16(0.003).tobytes(), np.uint8)
    else:
        blocks[:, 0:2] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
        blocks[:, 2:4] = np.frombuffer(np.float16(0.02).tobytes(), np.uint8)
    x = np.full((T, in_dim), 127.0, np.float32)
    x[1::2] *= -1
    x[:, ::7] = 126.0
    raw = blocks.reshape(-1)
    be.set_tuning("gemm_small_max_tokens", 1024)
    be.set_tuning("gemm_sb_waves", waves)
    try:
        got = be.matmul(x, T, qm(raw, t, in_dim, out_dim))
    finally:
        be.set_tuning("gemm_small_max_tokens", 1)
        be.set_tuning("gemm_sb_waves", 8)
    assert kname(be).startswith("ogm_gemm_sb_") and ("_w16_" in kname(be)) == (waves == 16)
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), "extreme ranges")


def test_mfma_gemm_rows_too_long_for_the_plane_kernel(be):
    """The Q4_K and Q5_K tiled kernels keep the tokens' scale of every super-block in LDS for the first pass;
    rows beyond 128 super-blocks (32768 values) are outside what the GEMM path accepts: they go through the
    multi-token GEMV in the GEMM's float order, with the same bits."""
    t, in_dim, out_dim, T = Q4_K, 33792, 40, 20
    raw = synth_weights(t, in_dim, out_dim, seed=4)
    x = synth_x(T, in_dim, seed=5)
    got = be.matmul(x, T, qm(raw, t, in_dim, out_dim))
    assert kname(be).startswith("ogm_gemv_kernel")
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), "long rows")
    got = be.matmul(x, T, qm(synth_weights(Q5_K, in_dim, out_dim, seed=6), Q5_K, in_dim, out_dim))
    assert kname(be).startswith("ogm_gemv_kernel")
    assert_bits(got, oracle.matmul(Q5_K, synth_weights(Q5_K, in_dim, out_dim, seed=6), in_dim, out_dim, x, T), "long rows, Q5_K")


@pytest.mark.parametrize("t,n_tokens,outs,kernel", [
    (Q4_K, 40, (300, 130, 64), "ogm_gemm_q4k_i8p_r64_kernel"),
    (Q4_K, 300, (6000, 3000, 2100), "ogm_gemm_q4k_i8p_kernel"),
    (Q5_K, 130, (520, 70, 129), "ogm_gemm_q5k_i8p_r64_kernel"),
    (Q5_K, 300, (6000, 3000, 2100), "ogm_gemm_q5k_i8p_kernel"),
    (Q6_K, 140, (300, 130, 64), "ogm_gemm_q6k_i8_r64_kernel"),
    (Q6_K, 300, (6000, 3000, 2100), "ogm_gemm_q6k_i8_kernel"),
    (Q3_K, 140, (128, 300, 70), "ogm_gemm_q3k_i8_r64_kernel"),
    (Q3_K, 300, (6000, 3000, 2100), "ogm_gemm_q3k_i8_kernel"),
    (Q4_K, 40, (300, 130, 64), "ogm_gemm_sb_q4k_kernel"),
    (Q5_K, 20, (520, 70, 129), "ogm_gemm_sb_q5k_kernel"),
    (Q6_K, 33, (300, 31), "ogm_gemm_sb_q6k_kernel"),
    (Q3_K, 33, (128, 300, 70), "ogm_gemm_sb_q3k_kernel"),
])
def test_k_quant_matrices_over_one_input_share_a_gemm_launch(be, t, n_tokens, outs, kernel):
    """q / k / v (llama.rs:730-746) at prefill widths: K-quant matrices of one type over the same
    activations go out as one launch whose row tiles run through the matrices in turn; every
    output bit equals the CPU GEMM's, ragged last tiles included."""
    from orangu_amd.hiprt import DeviceBuffer, device_synchronize
    in_dim = 512
    raws = [synth_weights(t, in_dim, od, seed=90 + i) for i, od in enumerate(outs)]
    hs = [be.upload_raw(r, t, in_dim, od) for r, od in zip(raws, outs)]
    x = synth_x(n_tokens, in_dim, seed=17)
    xd = DeviceBuffer.from_numpy(x)
    yds = [DeviceBuffer(4 * n_tokens * od) for od in outs]
    be.set_tuning("gemm_small_max_tokens", 1024 if "_sb_" in kernel else 1)
    try:
        be.matmul_multi_dev(hs, xd.ptr, n_tokens, [y.ptr for y in yds])
    finally:
        be.set_tuning("gemm_small_max_tokens", 1)
    device_synchronize()
    assert kname(be) == kernel
    for r, od, yd in zip(raws, outs, yds):
        want = oracle.matmul(t, r, in_dim, od, x, n_tokens)
        assert_bits(yd.to_numpy(np.float32, n_tokens * od), want, f"{od} rows of {outs}")
    for h in hs:
        be.free_weight(h)
    for b in [xd] + yds:
        b.free()


def test_mfma_gemm_equals_small_batch_kernel_and_is_batch_independent(be):
    """The two GPU kernels that serve ogm_matmul (multi-token GEMV below 9 tokens, MFMA GEMM above)
    must agree bit for bit, and a token's result must not depend on the batch (vecdot.rs:4522-4549)."""
    in_dim, out_dim = 2048, 48
    raw, _ = k_fixture(Q4_K, in_dim, out_dim, 1, 77)
    x = synth_x(40, in_dim, seed=5)
    w = qm(raw, Q4_K, in_dim, out_dim)
    full = be.matmul(x, 40, w).reshape(40, out_dim)
    be.set_tuning("gemm_min_tokens", 1000)
    try:
        small = be.matmul(x, 40, w).reshape(40, out_dim)
        assert kname(be).startswith("ogm_gemv_kernel")
    finally:
        be.set_tuning("gemm_min_tokens", GEMM_FROM)
    assert_bits(full, small, "mfma vs multi-token gemv")
    for n in (9, 17, 33):
        part = be.matmul(x[:n], n, w).reshape(n, out_dim)
        assert_bits(part, full[:n], f"{n} of 40")


@pytest.mark.parametrize("T", [16, 272])
@pytest.mark.parametrize("qs_lo,qs_hi,sign", [(0xFF, 0xFF, "alt"), (0x00, 0x00, "alt"), (0x0F, 0xF0, "pos"),
                                               (0xF0, 0x0F, "neg"), (0xFF, 0x00, "block")])
def test_mfma_gemm_adversarial_integer_ranges(be, qs_lo, qs_hi, sign, T):
    """Largest magnitudes the integer stage can see: nibbles 0 or 15, scales and mins 63, activations
    +-127.  The per-super-block sum reaches 3.1e7 > 2^24; the int8 kernels keep the whole sum in 32-bit
    integers and convert once (63 * 15 + 128 = 1073 split into the planes 4 and -79)."""
    in_dim, out_dim = 1024, 32
    blocks = np.zeros((out_dim * 4, 144), np.uint8)
    blocks[:, 0:2] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    blocks[:, 2:4] = np.frombuffer(np.float16(0.02).tobytes(), np.uint8)
    blocks[:, 4:16] = 0xFF
    blocks[:, 16:80] = qs_lo
    blocks[:, 80:] = qs_hi
    x = np.full((T, in_dim), 127.0, np.float32)
    if sign == "alt":
        x[1::2] *= -1
        x[:, ::7] = 126.0
    elif sign == "neg":
        x *= -1
    elif sign == "block":
        x[:, 128:256] *= -1
        x[3] = -127.0
    raw = blocks.reshape(-1)
    got = be.matmul(x, T, qm(raw, Q4_K, in_dim, out_dim))
    assert kname(be) == "ogm_gemm_q4k_i8p_r64_kernel"
    want = oracle.matmul(Q4_K, raw, in_dim, out_dim, x, T)
    assert_bits(got, want, "extreme ranges")
    isum, imin = be.dump_block_sums(x[0], 1, qm(raw, Q4_K, in_dim, out_dim))
    say("extreme isum", int(np.abs(isum).max()), "imin", int(np.abs(imin).max()))


@pytest.mark.parametrize("in_dim,out_dim,T", [
    (256, 5, 9), (512, 130, 17), (768, 64, 129), (1024, 100, 64), (1280, 257, 40), (2048, 37, 128),
    (4096, 200, 130), (14336, 96, 257), (4096, 1000, 512), (1792, 33, 10), (512, 4200, 513),
])
@pytest.mark.parametrize("variant", [0, 1])
def test_mfma_gemm_q6k_matches_cpu_gemm(be, in_dim, out_dim, T, variant):
    """Q6_K at n_tokens >= 9 takes an MFMA kernel; values must equal gemm_k_q6_k (vecdot.rs:2352-2398).
    The int8 kernel folds each scale into its weights and splits the 13-bit products into two int8 planes,
    on 128-row tiles or, when those are few, 64-row tiles (variant 1: always); every integer stays exact."""
    raw = synth_weights(Q6_K, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T + 1)
    w = qm(raw, Q6_K, in_dim, out_dim)
    say("gemm q6k", in_dim, out_dim, T, variant)
    tile_rows(be, 64 if variant == 1 else 0)
    try:
        got = be.matmul(x, T, w)
    finally:
        tile_rows(be, 0)
    small_grid = ((T + 127) // 128) * ((out_dim + 63) // 64) <= 256
    assert kname(be) == ("ogm_gemm_q6k_i8_r64_kernel" if variant == 1 or small_grid else "ogm_gemm_q6k_i8_kernel")
    want = oracle.matmul(Q6_K, raw, in_dim, out_dim, x, T)
    assert_close(got, want, "mfma gemm q6k")
    assert_bits(got, want, "mfma gemm q6k")
    be.set_tuning("gemm_min_tokens", 100000)
    try:
        small = be.matmul(x, T, w)
        assert kname(be).startswith("ogm_gemv_kernel")
    finally:
        be.set_tuning("gemm_min_tokens", GEMM_FROM)
    assert_bits(got, small, "mfma vs multi-token gemv")


@pytest.mark.parametrize("ql,qh,sc,sign", [(0xFF, 0xFF, 0x7F, "alt"), (0x00, 0x00, 0x80, "pos"), (0xFF, 0xFF, 0x80, "neg"),
                                           (0x00, 0x00, 0x7F, "alt"), (0xF0, 0x0F, 0x8F, "block"), (0x0F, 0xF0, 0x70, "pos")])
@pytest.mark.parametrize("variant", [0, 3])
def test_mfma_gemm_q6k_adversarial_integer_ranges(be, ql, qh, sc, sign, variant):
    """Extreme 6-bit values (0 -> -32, 63 -> +31), scales -128 / +127 / -113 / +112 and activations
    +-127: |isum| reaches 1.3e8, far past 2^24.  In the int8 kernels (variant 0: 64-row tiles on this small
    grid; variant 3: 128-row tiles, by way of 300 tokens x 6000 rows) -128 * -32 = 4096 is the product with the
    largest high plane, +16, and 256 H + L stays in 32 bits."""
    in_dim, out_dim, T = (1024, 6000, 300) if variant == 3 else (1024, 32, 16)
    blocks = np.zeros((out_dim * 4, 210), np.uint8)
    blocks[:, 0:128] = ql
    blocks[:, 128:192] = qh
    blocks[:, 192:208] = sc
    blocks[:, 208:210] = np.frombuffer(np.float16(0.003).tobytes(), np.uint8)
    x = np.full((T, in_dim), 127.0, np.float32)
    if sign == "alt":
        x[1::2] *= -1
        x[:, ::7] = 126.0
    elif sign == "neg":
        x *= -1
    elif sign == "block":
        x[:, 128:256] *= -1
        x[3] = -127.0
    raw = blocks.reshape(-1)
    got = be.matmul(x, T, qm(raw, Q6_K, in_dim, out_dim))
    assert kname(be) == {0: "ogm_gemm_q6k_i8_r64_kernel", 3: "ogm_gemm_q6k_i8_kernel"}[variant]
    want = oracle.matmul(Q6_K, raw, in_dim, out_dim, x, T)
    assert_bits(got, want, "extreme ranges")
    isum, _ = be.dump_block_sums(x[0], 1, qm(raw, Q6_K, in_dim, out_dim))
    say("extreme q6k isum", int(np.abs(isum).max()))


@pytest.mark.parametrize("t,kernel", [(Q3_K, "ogm_gemm_q3k_i8_kernel"), (Q5_K, "ogm_gemm_q5k_i8p_kernel")])
@pytest.mark.parametrize("in_dim,out_dim,T", [
    (256, 5, 9), (512, 130, 17), (768, 64, 129), (1024, 100, 64), (1280, 257, 40), (2048, 37, 128),
    (4096, 200, 130), (14336, 96, 257), (4096, 1000, 512), (1792, 33, 10), (512, 4200, 513),
])
def test_mfma_gemm_q3k_q5k_match_cpu_gemm(be, t, kernel, in_dim, out_dim, T):
    """Q3_K (a KKind::Q6K row, vecdot.rs:2100-2117) and Q5_K (a KKind::Q4K row, :2064-2088) on their int8
    kernels (planes of scale-folded weights, on 64-row tiles when those are few): every bit of gemm_k_q6_k /
    gemm_k_q4_k (vecdot.rs:2213-2255, 2352-2398), and of the multi-token GEMV."""
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T + 1)
    w = qm(raw, t, in_dim, out_dim)
    say("gemm", kernel, in_dim, out_dim, T)
    got = be.matmul(x, T, w)
    kernel = plane_kernel(kernel[:-len("_kernel")], T, out_dim)
    assert kname(be) == kernel
    want = oracle.matmul(t, raw, in_dim, out_dim, x, T)
    assert_close(got, want, kernel)
    assert_bits(got, want, kernel)
    be.set_tuning("gemm_min_tokens", 100000)
    try:
        small = be.matmul(x, T, w)
        assert kname(be).startswith("ogm_gemv_kernel")
    finally:
        be.set_tuning("gemm_min_tokens", GEMM_FROM)
    assert_bits(got, small, "mfma vs multi-token gemv")


@pytest.mark.parametrize("qs,qh,sc,sign", [(0xFF, 0xFF, 0xFF, "alt"), (0x00, 0x00, 0xFF, "pos"), (0xFF, 0xFF, 0xFF, "neg"),
                                           (0xFF, 0xFF, 0x3F, "block"), (0xF0, 0x55, 0xC7, "alt"), (0x0F, 0xAA, 0x00, "pos")])
def test_mfma_gemm_q5k_adversarial_integer_ranges(be, qs, qh, sc, sign):
    """Weights 0 and 31, scales and mins 63, activations +-127: a super-block's sum reaches
    63 * 31 * 127 * 256 = 6.3e7 and the mins' 63 * 8 * 4064 = 2.0e6; both planes' chains stay exact."""
    in_dim, out_dim, T = 1024, 32, 16
    blocks = np.zeros((out_dim * 4, 176), np.uint8)
    blocks[:, 0:2] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    blocks[:, 2:4] = np.frombuffer(np.float16(0.02).tobytes(), np.uint8)
    blocks[:, 4:16] = sc
    blocks[:, 16:48] = qh
    blocks[:, 48:176] = qs
    x = np.full((T, in_dim), 127.0, np.float32)
    if sign == "alt":
        x[1::2] *= -1
        x[:, ::7] = 126.0
    elif sign == "neg":
        x *= -1
    elif sign == "block":
        x[:, 128:256] *= -1
        x[3] = -127.0
    raw = blocks.reshape(-1)
    got = be.matmul(x, T, qm(raw, Q5_K, in_dim, out_dim))
    assert kname(be) == "ogm_gemm_q5k_i8p_r64_kernel"
    assert_bits(got, oracle.matmul(Q5_K, raw, in_dim, out_dim, x, T), "extreme ranges")
    isum, imin = be.dump_block_sums(x[0], 1, qm(raw, Q5_K, in_dim, out_dim))
    say("extreme q5k isum", int(np.abs(isum).max()), "imin", int(np.abs(imin).max()))


@pytest.mark.parametrize("qs,hm,sc,sign", [(0xFF, 0xFF, 0xFF, "alt"), (0x00, 0x00, 0x00, "pos"), (0x00, 0x00, 0xFF, "neg"),
                                           (0xFF, 0x00, 0x00, "block"), (0x1B, 0x5A, 0x9C, "alt"), (0xE4, 0xA5, 0x63, "pos")])
@pytest.mark.parametrize("variant", [0, 3])
def test_mfma_gemm_q3k_adversarial_integer_ranges(be, qs, hm, sc, sign, variant):
    """Weights -4 and 3, scales -32 and 31 (every six-bit pattern's bytes at their extremes) and
    activations +-127.  -32 * -4 = 128 is the product that does not fit an int8: the int8 kernels
    (variant 0: 64-row tiles on this small grid; 3: 128-row tiles, by way of 300 tokens x 6000 rows)
    carry the negated product, -128."""
    in_dim, out_dim, T = (1024, 6000, 300) if variant == 3 else (1024, 32, 16)
    blocks = np.zeros((out_dim * 4, 110), np.uint8)
    blocks[:, 0:32] = hm
    blocks[:, 32:96] = qs
    blocks[:, 96:108] = sc
    blocks[:, 108:110] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    x = np.full((T, in_dim), 127.0, np.float32)
    if sign == "alt":
        x[1::2] *= -1
        x[:, ::7] = 126.0
    elif sign == "neg":
        x *= -1
    elif sign == "block":
        x[:, 128:256] *= -1
        x[3] = -127.0
    raw = blocks.reshape(-1)
    got = be.matmul(x, T, qm(raw, Q3_K, in_dim, out_dim))
    assert kname(be) == {0: "ogm_gemm_q3k_i8_r64_kernel", 3: "ogm_gemm_q3k_i8_kernel"}[variant]
    assert_bits(got, oracle.matmul(Q3_K, raw, in_dim, out_dim, x, T), "extreme ranges")


# ---------------------------------------------------------------- grouped launches

@pytest.mark.parametrize("t", [Q8_0, Q5_0, Q4_0, IQ4_NL, Q3_K, Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("T,decode", [(1, False), (1, True), (4, True), (3, False), (16, False), (11, True)])
def test_grouped_weights_over_one_input_equal_single_calls(be, t, T, decode):
    """q/k/v and gate/up read one input (engine/arch/mod.rs:1082-1096): the grouped call equals
    matmul / matmul_decode per weight, also past four weights (two launches) and with ragged
    out_dims."""
    from orangu_amd.hiprt import DeviceBuffer, device_synchronize
    in_dim = 1024
    outs = [70, 16, 33, 128, 5]
    raws = [synth_weights(t, in_dim, od, seed=40 + i) for i, od in enumerate(outs)]
    ws = [qm(r, t, in_dim, od) for r, od in zip(raws, outs)]
    x = synth_x(T, in_dim, seed=T)
    xd = DeviceBuffer.from_numpy(x)
    yds = [DeviceBuffer(T * od * 4) for od in outs]
    say("grouped", t, T, decode)
    for yd in yds:
        yd.fill(0xFF)
    be.matmul_multi_dev([be.upload(w) for w in ws], xd.ptr, T, [yd.ptr for yd in yds], decode)
    device_synchronize()
    for raw, od, yd in zip(raws, outs, yds):
        got = yd.to_numpy(np.float32, T * od)
        want = (oracle.matmul_decode if decode else oracle.matmul)(t, raw, in_dim, od, x, T)
        assert_bits(got, want, f"out_dim {od}")
    for b in [xd] + yds:
        b.free()


def test_grouped_call_rejects_mixed_weights(be):
    from orangu_amd import OgmError
    from orangu_amd.hiprt import DeviceBuffer
    a = qm(synth_weights(Q4_K, 256, 4, seed=1), Q4_K, 256, 4)
    b = qm(synth_weights(Q6_K, 256, 4, seed=2), Q6_K, 256, 4)
    c = qm(synth_weights(Q4_K, 512, 4, seed=3), Q4_K, 512, 4)
    xd, yd = DeviceBuffer(512 * 4), DeviceBuffer(64)
    for pair in ((a, b), (a, c)):
        with pytest.raises(OgmError):
            be.matmul_multi_dev([be.upload(w) for w in pair], xd.ptr, 1, [yd.ptr, yd.ptr])
    xd.free()
    yd.free()


def test_matmul_batch_groups_ops_that_share_their_input(be):
    """Backend::matmul_batch over [wq, wk, wv] with one x (engine/arch/mod.rs:1082-1096): same
    values as the ops one by one, whatever the grouping."""
    from orangu_amd import MatmulOp
    in_dim = 2048
    x1, x4 = synth_x(1, in_dim, seed=5), synth_x(4, in_dim, seed=6)
    mk = lambda t, od, s: qm(synth_weights(t, in_dim, od, seed=s), t, in_dim, od)
    wq, wk, wv = mk(Q4_K, 96, 1), mk(Q4_K, 32, 2), mk(Q6_K, 32, 3)
    gate, up = mk(Q4_K, 200, 4), mk(Q4_K, 200, 5)
    ops = [MatmulOp(x1, 1, wq), MatmulOp(x1, 1, wk), MatmulOp(x1, 1, wv),
           MatmulOp(x4, 4, gate), MatmulOp(x4, 4, up), MatmulOp(x1.copy(), 1, gate)]
    for decode in (False, True):
        outs = (be.matmul_batch_decode if decode else be.matmul_batch)(ops)
        for op, y in zip(ops, outs):
            one = (be.matmul_decode if decode else be.matmul)(op.x, op.n_tokens, op.w)
            assert_bits(y, one, "grouped batch")
            want = (oracle.matmul_decode if decode else oracle.matmul)(
                op.w.ggml_type(), op.w.raw_bytes(), in_dim, op.w.out_dim, op.x, op.n_tokens)
            assert_bits(y, want, "grouped batch vs cpu")


def test_concurrent_callers_share_one_backend(be):
    """The scheduler calls a backend from one blocking-pool thread per slot (scheduler.rs:16-22):
    calls from several threads must serialise inside the library and each get their own result."""
    import threading
    in_dim = 1024
    ws = [(t, synth_weights(t, in_dim, od, seed=200 + i), od) for i, (t, od) in
          enumerate(((Q4_K, 300), (Q6_K, 130), (Q8_0, 257), (Q4_K, 64)))]
    mats = [qm(raw, t, in_dim, od) for t, raw, od in ws]
    xs = [synth_x(T, in_dim, seed=300 + i) for i, T in enumerate((1, 3, 12, 40))]
    want = {(i, j): oracle.matmul(ws[i][0], ws[i][1], in_dim, ws[i][2], xs[j], xs[j].shape[0]).reshape(-1)
            for i in range(4) for j in range(4)}
    for m in mats:
        be.upload(m)
    errors = []

    def worker(k):
        try:
            for rep in range(6):
                i, j = (k + rep) % 4, (k * 3 + rep) % 4
                got = be.matmul(xs[j].reshape(-1), xs[j].shape[0], mats[i])
                if not np.array_equal(got.view(np.uint32), want[(i, j)].view(np.uint32)):
                    errors.append((k, rep, i, j))
        except Exception as e:  # noqa: BLE001
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


def test_host_calls_on_pinned_buffers_and_through_device_copies_agree(be):
    """A host-pointer call of up to 512 KiB runs its kernels on the pinned staging buffers in place
    (host_zero_copy 1, the default); larger calls, and all of them with host_zero_copy 0, go through
    device copies.  Same bits either way, for one GEMV, a small GEMM, a batch over a shared input and a
    call just past the limit."""
    from orangu_amd import MatmulOp
    in_dim = 1024
    wa, wb = synth_weights(Q4_K, in_dim, 300, seed=41), synth_weights(Q6_K, in_dim, 130, seed=42)
    ma, mb = qm(wa, Q4_K, in_dim, 300), qm(wb, Q6_K, in_dim, 130)
    x1, x7, x100 = synth_x(1, in_dim, 43), synth_x(7, in_dim, 44), synth_x(100, in_dim, 45)   # 100 tokens: 529 KiB
    res = {}
    for zc in (1, 0):
        be.set_tuning("host_zero_copy", zc)
        try:
            ops = [MatmulOp(x7.reshape(-1), 7, ma), MatmulOp(x7.reshape(-1), 7, mb), MatmulOp(x1.reshape(-1), 1, mb)]
            res[zc] = [be.matmul(x1.reshape(-1), 1, ma), be.matmul_decode(x7.reshape(-1), 7, mb),
                       be.matmul(x7.reshape(-1), 7, ma), be.matmul(x100.reshape(-1), 100, ma),
                       *be.matmul_batch(ops), *be.matmul_batch_decode(ops)]
        finally:
            be.set_tuning("host_zero_copy", 1)
    for a, b in zip(res[1], res[0]):
        assert_bits(a, b, "pinned in place vs device copies")
    assert_bits(res[1][0], oracle.matmul(Q4_K, wa, in_dim, 300, x1, 1), "GEMV on pinned buffers")
    assert_bits(res[1][2], oracle.matmul(Q4_K, wa, in_dim, 300, x7, 7), "small GEMM on pinned buffers")
    assert_bits(res[1][5], oracle.matmul(Q6_K, wb, in_dim, 130, x7, 7), "batch on pinned buffers")


@pytest.mark.parametrize("sign", ["pos", "alt"])
def test_q5k_extreme_integer_ranges(be, sign):
    """Q5_K's largest magnitudes: every weight 31, scales and mins 63, activations +-127: isum
    reaches 6.3e7 per super-block (vecdot.rs:3077), inside i32; GEMV, decode batch and multi-token
    matmul all give the CPU path's bits."""
    in_dim, out_dim, T = 1024, 20, 12
    blocks = np.zeros((out_dim * 4, 176), np.uint8)
    blocks[:, 0:2] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    blocks[:, 2:4] = np.frombuffer(np.float16(0.02).tobytes(), np.uint8)
    blocks[:, 4:] = 0xFF
    x = np.full((T, in_dim), 127.0, np.float32)
    if sign == "alt":
        x[1::2] *= -1
        x[:, ::7] = -126.0
    raw = blocks.reshape(-1)
    w = qm(raw, Q5_K, in_dim, out_dim)
    isum, imin = be.dump_block_sums(x[0], 1, w)
    wi, wm = oracle.block_sums(Q5_K, raw, in_dim, out_dim, x[0], 1)
    assert np.array_equal(isum, wi) and np.array_equal(imin, wm)
    say("extreme q5k isum", int(np.abs(isum).max()), "imin", int(np.abs(imin).max()))
    assert_bits(be.matmul(x[0], 1, w), oracle.matmul(Q5_K, raw, in_dim, out_dim, x[0], 1), "gemv")
    assert_bits(be.matmul(x, T, w), oracle.matmul(Q5_K, raw, in_dim, out_dim, x, T), "matmul")
    assert_bits(be.matmul_decode(x, T, w), oracle.matmul_decode(Q5_K, raw, in_dim, out_dim, x, T), "decode")


@pytest.mark.parametrize("hmask,qs", [(0x00, 0x00), (0x00, 0xFF), (0xFF, 0xFF)])
def test_q3k_extreme_integer_ranges(be, hmask, qs):
    """Q3_K's poles: weights -4 (hmask clear, bits 0), -1 and 3, every scale byte 0xFF (scales
    63 - 32 = 31) or 0x00 (-32), activations +-127: |isum| up to 4.2e6 (vecdot.rs:3271-3272)."""
    in_dim, out_dim, T = 1024, 20, 12
    for scb in (0xFF, 0x00):
        blocks = np.zeros((out_dim * 4, 110), np.uint8)
        blocks[:, 0:32] = hmask
        blocks[:, 32:96] = qs
        blocks[:, 96:108] = scb
        blocks[:, 108:110] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
        x = np.full((T, in_dim), 127.0, np.float32)
        x[1::2] *= -1
        x[:, ::7] = -126.0
        raw = blocks.reshape(-1)
        w = qm(raw, Q3_K, in_dim, out_dim)
        isum, _ = be.dump_block_sums(x[0], 1, w)
        wi, _ = oracle.block_sums(Q3_K, raw, in_dim, out_dim, x[0], 1)
        assert np.array_equal(isum, wi)
        say("extreme q3k isum", int(np.abs(isum).max()))
        assert_bits(be.matmul(x[0], 1, w), oracle.matmul(Q3_K, raw, in_dim, out_dim, x[0], 1), "gemv")
        assert_bits(be.matmul(x, T, w), oracle.matmul(Q3_K, raw, in_dim, out_dim, x, T), "matmul")
        assert_bits(be.matmul_decode(x, T, w), oracle.matmul_decode(Q3_K, raw, in_dim, out_dim, x, T), "decode")


@pytest.mark.parametrize("t", [Q4_0, Q5_0, IQ4_NL])
def test_per_32_nibble_types_every_byte_value_and_extreme_sums(be, t):
    """Every nibble pair (and, for Q5_0, both values of every fifth bit) against activations of
    +-127: the per-32 integer sums reach 32 * 127 * 127 (IQ4_NL), 32 * 16 * 127 (Q5_0)."""
    bb = BLOCK[t][0]
    in_dim, out_dim = 256, 64
    blocks = np.zeros((out_dim * 8, bb), np.uint8)
    blocks[:, 0:2] = np.frombuffer(np.float16(0.03125).tobytes(), np.uint8)
    vals = np.arange(out_dim * 8 * 16, dtype=np.uint32)
    blocks[:, bb - 16:] = ((vals * 37 + (vals >> 4) * 11) & 0xFF).reshape(-1, 16).astype(np.uint8)
    blocks[::5, bb - 16:] = 0x00      # zero point / level 0 everywhere
    blocks[1::5, bb - 16:] = 0xFF
    if t == Q5_0:
        blocks[:, 2:6] = ((vals[::16] * 2654435761) >> 3).astype(np.uint32).view(np.uint8).reshape(-1, 4)
        blocks[::5, 2:6] = 0x00
        blocks[1::5, 2:6] = 0xFF
    raw = blocks.reshape(-1)
    for sign in (1.0, -1.0):
        x = np.full((3, in_dim), 127.0 * sign, np.float32)
        x[1, ::2] *= -1
        x[2, ::3] = 63.0
        w = qm(raw, t, in_dim, out_dim)
        isum, _ = be.dump_block_sums(x, 3, w)
        wi, _ = oracle.block_sums(t, raw, in_dim, out_dim, x, 3)
        assert np.array_equal(isum, wi)
        say("per-32 extreme isum", t, int(np.abs(isum).max()))
        assert_bits(be.matmul(x[0], 1, w), oracle.matmul(t, raw, in_dim, out_dim, x[0], 1), "gemv")
        assert_bits(be.matmul(x, 3, w), oracle.matmul(t, raw, in_dim, out_dim, x, 3), "matmul")


@pytest.mark.parametrize("t", [Q8_0, Q5_0, Q4_0, IQ4_NL])
@pytest.mark.parametrize("in_dim,out_dim,T", [(64, 5, 9), (128, 130, 17), (896, 64, 40), (4096, 257, 130),
                                              (4864, 100, 300), (1024, 128, 128), (2048, 129, 513)])
def test_mfma_gemm_flat_types_match_cpu_gemm(be, t, in_dim, out_dim, T):
    """The symmetric per-32 types at n_tokens >= 9 and in_dim % 64 == 0 take the MFMA flat GEMM; values
    must equal dot_flat_pair (vecdot.rs:2598-2629) bit for bit, and the small-batch kernel's."""
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim + T + t)
    x = synth_x(T, in_dim, seed=T + 1)
    w = qm(raw, t, in_dim, out_dim)
    say("flat gemm", t, in_dim, out_dim, T)
    got = be.matmul(x, T, w)
    assert kname(be) == "ogm_gemm_flat_kernel"
    want = oracle.matmul(t, raw, in_dim, out_dim, x, T)
    assert_close(got, want, "flat mfma gemm")
    assert_bits(got, want, "flat mfma gemm")
    be.set_tuning("gemm_min_tokens", 100000)
    try:
        small = be.matmul(x, T, w)
        assert kname(be).startswith("ogm_gemv_kernel")
    finally:
        be.set_tuning("gemm_min_tokens", GEMM_FROM)
    assert_bits(small, want, "multi-token gemv")


@pytest.mark.parametrize("waves", [8, 16])
@pytest.mark.parametrize("t", [Q8_0, Q5_0, Q4_0, IQ4_NL])
@pytest.mark.parametrize("in_dim,out_dim,T", [(64, 5, 9), (128, 130, 17), (896, 64, 40), (4096, 257, 130), (4864, 100, 33),
                                              (1024, 128, 128), (2048, 129, 70), (14336, 70, 45), (512, 31, 2)])
def test_small_batch_flat_types_match_cpu_gemm(be, t, in_dim, out_dim, T, waves):
    """The per-32 types' small-batch kernel (32 rows x 32 tokens a workgroup, its eight or sixteen waves on different
    blocks, a block one int8 matrix instruction, the blocks' terms added in ascending order after every round of two
    blocks a wave): every bit of dot_flat_pair (vecdot.rs:2598-2629), with rows, tokens and blocks that do not fill
    the last workgroup or the last round.  (Sixteen waves keep one round's activation scales in LDS at a time.)"""
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim + T + t)
    x = synth_x(T, in_dim, seed=T + 1)
    w = qm(raw, t, in_dim, out_dim)
    be.set_tuning("gemm_small_max_tokens", 1024)
    be.set_tuning("gemm_min_tokens", 2)
    be.set_tuning("gemm_sb_waves", waves)
    try:
        got = be.matmul(x, T, w)
        w16 = waves == 16
        assert kname(be) == ("ogm_gemm_sb_flat_w16_kernel" if w16 else "ogm_gemm_sb_flat_kernel")
    finally:
        be.set_tuning("gemm_small_max_tokens", 1)
        be.set_tuning("gemm_min_tokens", GEMM_FROM)
        be.set_tuning("gemm_sb_waves", 0)
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), "small-batch flat gemm")


@pytest.mark.parametrize("t", [Q8_0, Q5_0, Q4_0, IQ4_NL])
def test_small_batch_flat_extreme_block_sums(be, t):
    """As test_mfma_gemm_flat_extreme_block_sums, through the small-batch kernel: 32 * 127 * 127 per block in the
    int8 matrix instruction's 32-bit sums."""
    bb = BLOCK[t][0]
    in_dim, out_dim, T = 256, 40, 24
    blocks = np.zeros((out_dim * 8, bb), np.uint8)
    blocks[:, 0:2] = np.frombuffer(np.float16(0.0078125).tobytes(), np.uint8)
    blocks[0::3, 2:] = 0x00 if t != Q8_0 else 0x81
    blocks[1::3, 2:] = 0xFF if t != Q8_0 else 0x7F
    blocks[2::3, 2:] = 0xF0 if t != Q8_0 else 0x81
    raw = blocks.reshape(-1)
    x = np.full((T, in_dim), 127.0, np.float32)
    x[1::2] *= -1
    x[:, 5::11] = -127.0
    be.set_tuning("gemm_small_max_tokens", 1024)
    try:
        got = be.matmul(x, T, qm(raw, t, in_dim, out_dim))
        assert kname(be) == "ogm_gemm_sb_flat_kernel"
    finally:
        be.set_tuning("gemm_small_max_tokens", 1)
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), "extreme sums, small-batch kernel")


@pytest.mark.parametrize("t", [Q8_0, Q5_0, Q4_0, IQ4_NL])
def test_mfma_gemm_flat_extreme_block_sums(be, t):
    """Largest per-32 sums: weights at their extremes against activations of +-127 (Q8_0 and IQ4_NL:
    32 * 127 * 127 = 516 128, exact in the f32 accumulator)."""
    bb = BLOCK[t][0]
    in_dim, out_dim, T = 256, 40, 24
    blocks = np.zeros((out_dim * 8, bb), np.uint8)
    blocks[:, 0:2] = np.frombuffer(np.float16(0.0078125).tobytes(), np.uint8)
    blocks[0::3, 2:] = 0x00 if t != Q8_0 else 0x81      # -127 / zero point / level 0
    blocks[1::3, 2:] = 0xFF if t != Q8_0 else 0x7F      # +127 / top level
    blocks[2::3, 2:] = 0xF0 if t != Q8_0 else 0x81
    raw = blocks.reshape(-1)
    x = np.full((T, in_dim), 127.0, np.float32)
    x[1::2] *= -1
    x[:, 5::11] = -127.0
    w = qm(raw, t, in_dim, out_dim)
    got = be.matmul(x, T, w)
    assert kname(be) == "ogm_gemm_flat_kernel"
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), "extreme sums")
    isum, _ = be.dump_block_sums(x[0], 1, w)
    say("flat extreme isum", t, int(np.abs(isum).max()))

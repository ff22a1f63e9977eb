"""Q5_1, Q2_K and IQ4_XS on the device against the CPU restatement: bit-exact through every entry point
(one token, decode batches, matmul of several tokens in the reference's several-token arithmetic), the
integer stage, the extremes of the integer ranges, full-size shapes, and the rows an embedding lookup reads."""
import numpy as np
import pytest

import oracle
from helpers import (BLOCK, IQ4_XS, Q2_K, Q3_K, Q4_K, Q5_1, Q5_K, Q6_K, activations_t, pin_scales, pseudo_bytes_fast,
                     row_bytes, synth_weights, synth_x)

pytestmark = pytest.mark.gpu
NEW = [Q5_1, Q2_K, IQ4_XS]


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def be():
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()  # raises if the HIP library or the device is missing: no fallback
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


@pytest.mark.parametrize("t", NEW)
def test_types_are_supported_and_round_trip(be, t):
    """supports (vecdot.rs:274-283) and unrepack(repack(W)) == W through the device."""
    bb, bel = BLOCK[t]
    assert be.supports_type(t)
    in_dim, out_dim = bel * 5, 77
    raw = np.random.default_rng(t).integers(0, 256, row_bytes(t, in_dim) * out_dim, dtype=np.uint8)
    assert np.array_equal(be.download(qm(raw, t, in_dim, out_dim)), raw)


@pytest.mark.parametrize("t,in_dim,out_dim", [
    (Q5_1, 32, 5), (Q5_1, 896, 19), (Q5_1, 4096, 130), (Q5_1, 4864, 7),
    (Q2_K, 256, 6), (Q2_K, 512, 5), (Q2_K, 4096, 130), (Q2_K, 5632, 33),
    (IQ4_XS, 256, 4), (IQ4_XS, 512, 5), (IQ4_XS, 4096, 130), (IQ4_XS, 5632, 33)])
def test_one_token_and_decode_batches_are_bit_exact(be, t, in_dim, out_dim):
    """dot_q5_1 / dot_k_row_q2_k / dot_k_row_iq4_xs (vecdot.rs:2886-2899, 3296-3318, 3245-3266) through matmul at
    one token and matmul_decode at 1..9 tokens (cpu.rs:265-317: each row of the batch is the one-token result)."""
    raw = pin_scales(pseudo_bytes_fast(row_bytes(t, in_dim) * out_dim, in_dim + out_dim), t)
    w = qm(raw, t, in_dim, out_dim)
    x = np.concatenate([activations_t(in_dim, k) for k in range(9)])
    say("new type", t, in_dim, out_dim)
    assert_bits(be.matmul(x[:in_dim], 1, w), oracle.matmul(t, raw, in_dim, out_dim, x[:in_dim], 1), "one token")
    for T in (1, 2, 5, 9):
        got = be.matmul_decode(x[:T * in_dim], T, w)
        assert_bits(got, oracle.matmul_decode(t, raw, in_dim, out_dim, x[:T * in_dim], T), f"decode batch of {T}")


@pytest.mark.parametrize("t,in_dim,out_dim", [
    (Q5_1, 64, 17), (Q5_1, 896, 33), (Q5_1, 4096, 70),
    (Q2_K, 512, 5), (Q2_K, 1024, 70), (Q2_K, 4096, 33),
    (IQ4_XS, 512, 5), (IQ4_XS, 1024, 70), (IQ4_XS, 4096, 33)])
@pytest.mark.parametrize("T", [2, 3, 7, 17, 130])
def test_matmul_of_several_tokens_is_bit_exact(be, t, in_dim, out_dim, T):
    """matmul at n_tokens > 1 (cpu.rs:55-167): IQ4_XS the K GEMM (gemm_k_iq4_xs, vecdot.rs:2305-2322: ad * (d * isum)),
    Q5_1 and Q2_K the rows-unpacked-once path over per-32 activations (vecdot.rs:1302-1314, 1144-1164, 1684-1745) --
    for Q2_K a different quantization and a term per group of 16.  Token counts cover the tile of four and its tail
    (the reference's cross_check_n_tokens shapes, vulkan/tests.rs:2612-2683)."""
    raw = synth_weights(t, in_dim, out_dim, seed=t * 1000 + in_dim + T)
    x = synth_x(T, in_dim, seed=T + 3)
    got = be.matmul(x, T, qm(raw, t, in_dim, out_dim))
    say("new type matmul", t, in_dim, out_dim, T, be.last_kernel())
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), "several tokens")


@pytest.mark.parametrize("t", NEW)
def test_integer_stage_is_exact(be, t):
    """The per-block integer sums of the one-token path against the CPU's."""
    in_dim, out_dim, T = 1024, 9, 3
    raw = pin_scales(pseudo_bytes_fast(row_bytes(t, in_dim) * out_dim, 77), t)
    x = synth_x(T, in_dim, seed=5)
    isum, imin = be.dump_block_sums(x, T, qm(raw, t, in_dim, out_dim))
    wi, wm = oracle.block_sums(t, raw, in_dim, out_dim, x, T)
    assert np.array_equal(isum, wi)
    if t == Q2_K:
        assert np.array_equal(imin, wm)


@pytest.mark.parametrize("t", NEW)
@pytest.mark.parametrize("sign", ["pos", "neg", "alt"])
def test_extreme_integer_ranges(be, t, sign):
    """Every quant at its largest magnitude with the largest scales against activations of +-127: Q5_1 31 * 127 per
    element (and the largest block sum for its m term), Q2_K scale and min 15 with quants 3, IQ4_XS level -127 with
    scale -32 (|isum| 32 * 127 * 127 * 256 = 1.3e8, inside i32)."""
    in_dim, out_dim, T = 1024, 7, 4
    bb, be_ = BLOCK[t]
    blocks = np.zeros((out_dim * in_dim // be_, bb), np.uint8)
    half = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    if t == Q5_1:
        blocks[:, 0:2], blocks[:, 2:4] = half, np.frombuffer(np.float16(-0.37).tobytes(), np.uint8)
        blocks[:, 4:] = 0xFF
    elif t == Q2_K:
        blocks[:, 0:80] = 0xFF
        blocks[:, 80:82], blocks[:, 82:84] = half, half
    else:
        blocks[:, 0:2] = half
        blocks[:, 2:8] = 0      # ls = 0 - 32 = -32 for every sub-block
        blocks[:, 8:] = 0       # index 0: level -127
    x = np.full((T, in_dim), 127.0, np.float32)
    if sign == "neg":
        x *= -1
    elif sign == "alt":
        x[:, 1::2] *= -1
        x[1] = -127.0
    raw = blocks.reshape(-1)
    w = qm(raw, t, in_dim, out_dim)
    assert_bits(be.matmul(x[0], 1, w), oracle.matmul(t, raw, in_dim, out_dim, x[0], 1), "extremes, one token")
    assert_bits(be.matmul(x, T, w), oracle.matmul(t, raw, in_dim, out_dim, x, T), "extremes, several tokens")
    assert_bits(be.matmul_decode(x, T, w), oracle.matmul_decode(t, raw, in_dim, out_dim, x, T), "extremes, decode batch")


@pytest.mark.parametrize("t,in_dim,out_dim", [(Q5_1, 4096, 4096), (Q2_K, 4096, 14336), (IQ4_XS, 14336, 4096),
                                              (IQ4_XS, 4096, 14336)])
def test_full_size_shapes(be, t, in_dim, out_dim):
    """The benchmark's FFN shapes at one token, bit for bit, and at 8 tokens on sampled rows."""
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + t)
    x = synth_x(8, in_dim, seed=2)
    w = qm(raw, t, in_dim, out_dim)
    assert_bits(be.matmul(x[0], 1, w), oracle.matmul(t, raw, in_dim, out_dim, x[0], 1), "full size, one token")
    got = np.asarray(be.matmul(x, 8, w)).reshape(8, out_dim)
    rows = np.r_[0:16, out_dim // 2:out_dim // 2 + 16, out_dim - 16:out_dim]
    rb = row_bytes(t, in_dim)
    sub = np.concatenate([raw[r * rb:(r + 1) * rb] for r in rows])
    assert_bits(got[:, rows], oracle.matmul(t, sub, in_dim, rows.size, x, 8), "full size, 8 tokens, sampled rows")
    be.evict(w)


@pytest.mark.parametrize("t", NEW)
def test_dequantized_rows_match_the_cpu_dequantizer(be, t):
    """The rows an embedding lookup reads (llama.rs:609-614 over quant.rs:615-636, 798-827, 1350-1375)."""
    in_dim, out_dim = 1024, 37
    raw = pin_scales(pseudo_bytes_fast(row_bytes(t, in_dim) * out_dim, 11), t)
    got = be.dequant_rows(qm(raw, t, in_dim, out_dim), 3, 20)
    rb = row_bytes(t, in_dim)
    want = np.stack([oracle.dequantize(t, raw[r * rb:(r + 1) * rb], in_dim) for r in range(3, 23)])
    assert_bits(got, want, "dequantized rows")


def test_q5_1_min_term_is_added_not_subtracted_on_the_device(be):
    """vecdot.rs:4195-4218 through the device: d = 0, m = 2.5 makes every weight 2.5; one token, a decode batch and
    matmul of several tokens give 2.5 * sum(x_q) * scale_x, bit for bit what the CPU restatement gives."""
    block = np.concatenate([np.frombuffer(np.float16(0.0).tobytes(), np.uint8), np.frombuffer(np.float16(2.5).tobytes(), np.uint8),
                            np.zeros(4, np.uint8), np.zeros(16, np.uint8)])
    raw = np.tile(block, 4 * 3)   # three rows of four blocks
    w = qm(raw, Q5_1, 128, 3)
    x = np.concatenate([activations_t(128, k) for k in range(3)])
    one = be.matmul(x[:128], 1, w)
    q, d, _ = oracle.quantize_act(x[:128])
    known = float(sum(np.float64(2.5) * d[b] * q[32 * b:32 * b + 32].astype(np.int64).sum() for b in range(4)))
    assert np.allclose(np.asarray(one, np.float64), known, rtol=1e-5, atol=1e-6), (one, known)
    assert_bits(one, oracle.matmul(Q5_1, raw, 128, 3, x[:128], 1), "one token")
    assert_bits(be.matmul_decode(x, 3, w), oracle.matmul_decode(Q5_1, raw, 128, 3, x, 3), "decode batch")
    assert_bits(be.matmul(x, 3, w), oracle.matmul(Q5_1, raw, 128, 3, x, 3), "several tokens")


def test_q2_k_two_step_calls_in_both_activation_modes(be):
    """The two-step path (quantize once, multiply several weights) for Q2_K at several tokens: matmul runs over per-32
    activations (cpu.rs:113-163), matmul_decode over per-256 ones (cpu.rs:265-317), so each has a quantize step of its
    own; a matmul step over the other mode's activations is refused and says which step it needs."""
    from orangu_amd import OgmError, hiprt
    in_dim, out_dim, T = 1024, 37, 3
    raw = synth_weights(Q2_K, in_dim, out_dim, seed=71)
    x = synth_x(T, in_dim, seed=72)
    h = be.upload_raw(raw, Q2_K, in_dim, out_dim)
    xd, yd = hiprt.DeviceBuffer.from_numpy(x), hiprt.DeviceBuffer(4 * T * out_dim)
    try:
        for decode, ref in ((True, oracle.matmul_decode), (False, oracle.matmul)):
            yd.fill(0xFF)
            hiprt.device_synchronize()   # (the fill runs on another stream than the library's)
            be.act_quantize_dev(Q2_K, xd.ptr, in_dim, T, decode=decode)
            be.matmul_act_dev(h, T, yd.ptr, decode)
            hiprt.device_synchronize()
            assert_bits(yd.to_numpy(np.float32, T * out_dim), ref(Q2_K, raw, in_dim, out_dim, x, T),
                        f"two-step Q2_K, decode={decode}")
            with pytest.raises(OgmError, match="ogm_act_quantize_decode_dev"):
                be.matmul_act_dev(h, T, yd.ptr, not decode)
    finally:
        be.free_weight(h)
        xd.free()
        yd.free()


@pytest.mark.parametrize("in_dim,out_dim,T,interleave,kernel", [
    (256, 5, 32, 1, "ogm_gemm_iq4xs_dma_kernel"), (1024, 130, 45, 2, "ogm_gemm_iq4xs_dmx_kernel"),
    (768, 257, 129, 1, "ogm_gemm_iq4xs_dma_kernel"), (2048, 129, 300, 2, "ogm_gemm_iq4xs_dmx_kernel"),
    (512, 4200, 513, 0, "ogm_gemm_iq4xs_dmx_kernel"), (256, 16600, 130, 0, "ogm_gemm_iq4xs_dma_kernel"),
    (14336, 70, 33, 2, "ogm_gemm_iq4xs_dmx_kernel"), (1280, 64, 31, 1, "ogm_gemm_iq4xs_dma_kernel"),
    (512, 200, 17, 0, "ogm_gemm_iq4xs_dmx_kernel"), (768, 3000, 20, 0, "ogm_gemm_iq4xs_dmx_kernel"),
    (256, 33000, 23, 0, "ogm_gemm_iq4xs_dma_kernel"), (1280, 64, 16, 0, "ogm_gemv_kernel<FmtIQ4XS,gemm>")])
def test_iq4_xs_batches_on_the_plane_kernels(be, in_dim, out_dim, T, interleave, kernel):
    """From seventeen tokens on (three passes of the GEMV kernel) IQ4_XS takes the GEMM kernels over prebuilt int8 planes (the scale of a sub-block of 32
    folded into IQ4_NL's levels, split by bytes as Q6_K's are; no other GEMM kernel knows the type): every bit of
    gemm_k_iq4_xs (vecdot.rs:2305-2322), on 128-row tiles and on the 64-row tiles with the f32 step between the
    matrix instructions (launches of up to 512 workgroups, by default); up to sixteen tokens the GEMV kernel in the same
    float order."""
    raw = synth_weights(IQ4_XS, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T)
    be.set_tuning("gemm_interleave", interleave)
    be.set_tuning("gemm_small_max_tokens", 1)   # (its small-batch kernel has a test of its own)
    try:
        got = be.matmul(x, T, qm(raw, IQ4_XS, in_dim, out_dim))
        assert be.last_kernel() == kernel
    finally:
        be.set_tuning("gemm_interleave", 0)
        be.set_tuning("gemm_small_max_tokens", 0)
    assert_bits(got, oracle.matmul(IQ4_XS, raw, in_dim, out_dim, x, T), "IQ4_XS over planes")


def test_iq4_xs_extreme_sums_on_the_plane_kernels(be):
    """Levels -127 and 113 under scales -32 and 31 against activations of +-127: the folded weights reach +-4064
    (planes -16 .. 16 and their low bytes), a super-block's sum 1.3e8."""
    in_dim, out_dim, T = 1024, 70, 40
    blocks = np.zeros((out_dim * 4, 136), np.uint8)
    blocks[:, 0:2] = np.frombuffer(np.float16(0.002).tobytes(), np.uint8)
    blocks[0::2, 2:4] = 0xFF      # scales_h: the two high bits of every scale set
    blocks[0::2, 4:8] = 0xFF      # scales_l: 63 - 32 = 31
    blocks[1::2, 2:8] = 0x00      # 0 - 32 = -32
    blocks[0::3, 8:] = 0x00       # level -127
    blocks[1::3, 8:] = 0xFF       # level 113
    blocks[2::3, 8:] = 0xF0
    raw = blocks.reshape(-1)
    x = np.full((T, in_dim), 127.0, np.float32)
    x[1::2] *= -1
    x[:, 5::11] = -127.0
    for interleave, small_max in ((1, 1), (2, 1), (0, 1024)):   # the two plane kernels, the small-batch kernel
        be.set_tuning("gemm_interleave", interleave)
        be.set_tuning("gemm_small_max_tokens", small_max)
        try:
            got = be.matmul(x, T, qm(raw, IQ4_XS, in_dim, out_dim))
            assert ("iq4xs_dm" if small_max == 1 else "sb_iq4xs") in be.last_kernel()
        finally:
            be.set_tuning("gemm_interleave", 0)
            be.set_tuning("gemm_small_max_tokens", 0)
        assert_bits(got, oracle.matmul(IQ4_XS, raw, in_dim, out_dim, x, T), f"extreme sums, {be.last_kernel()}")


@pytest.mark.parametrize("waves", [8, 16])
@pytest.mark.parametrize("in_dim,out_dim,T", [(256, 5, 9), (1024, 100, 17), (768, 64, 32), (1280, 257, 40), (14336, 96, 33),
                                              (2304, 130, 100), (256, 1, 300)])
def test_iq4_xs_small_batch_kernel(be, in_dim, out_dim, T, waves):
    """The K-quants' small-batch kernel with IQ4_XS's unpacking (32 rows x 32 tokens, the waves on different
    super-blocks, terms added in ascending order): every bit of gemm_k_iq4_xs (vecdot.rs:2305-2322)."""
    raw = synth_weights(IQ4_XS, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T + 2)
    be.set_tuning("gemm_small_max_tokens", 1024)
    be.set_tuning("gemm_sb_waves", waves)
    try:
        got = be.matmul(x, T, qm(raw, IQ4_XS, in_dim, out_dim))
        assert be.last_kernel() == ("ogm_gemm_sb_iq4xs_w16_kernel" if waves == 16 else "ogm_gemm_sb_iq4xs_kernel")
    finally:
        be.set_tuning("gemm_small_max_tokens", 0)
        be.set_tuning("gemm_sb_waves", 0)
    assert_bits(got, oracle.matmul(IQ4_XS, raw, in_dim, out_dim, x, T), "IQ4_XS small batch")


def test_iq4_xs_default_routing(be):
    """Up to eight tokens the GEMV kernel, then the small-batch kernel, and the plane kernels where a launch has
    enough workgroups for them."""
    raw = synth_weights(IQ4_XS, 512, 4200, seed=3)
    x = synth_x(300, 512, seed=4)
    w = qm(raw, IQ4_XS, 512, 4200)
    want = oracle.matmul(IQ4_XS, raw, 512, 4200, x, 300).reshape(300, 4200)
    for T, kernel in ((8, "ogm_gemv_kernel"), (9, "ogm_gemm_sb_iq4xs"), (64, "ogm_gemm_sb_iq4xs"), (300, "ogm_gemm_iq4xs_dmx_kernel")):
        got = be.matmul(x[:T], T, w)
        assert be.last_kernel().startswith(kernel), (T, be.last_kernel())
        assert_bits(got, want[:T], f"IQ4_XS, {T} tokens")


def test_iq4_xs_without_room_for_planes_stays_on_the_gemv_kernel(be):
    """With no memory allowed for planes the batch runs on the GEMV kernel in the GEMM's float order: same bits."""
    in_dim, out_dim, T = 512, 300, 700
    raw = synth_weights(IQ4_XS, in_dim, out_dim, seed=77)
    x = synth_x(T, in_dim, seed=78)
    be.set_tuning("gemm_plane_cache_mb", 0)
    try:
        got = be.matmul(x, T, qm(raw, IQ4_XS, in_dim, out_dim))
        assert be.last_kernel().startswith("ogm_gemv_kernel")
    finally:
        be.set_tuning("gemm_plane_cache_mb", 32768)
    assert_bits(got, oracle.matmul(IQ4_XS, raw, in_dim, out_dim, x, T), "IQ4_XS, no planes")


@pytest.mark.parametrize("in_dim,out_dim,T,kernel", [
    (64, 5, 9, "ogm_gemm_sb_flat_kernel"), (128, 130, 17, "ogm_gemm_sb_flat_kernel"), (896, 64, 40, "ogm_gemm_sb_flat_kernel"),
    (4864, 100, 33, "ogm_gemm_sb_flat_w16_kernel"), (2048, 129, 300, "ogm_gemm_sb_flat_w16_kernel"),
    (14336, 70, 45, "ogm_gemm_sb_flat_w16_kernel"), (512, 31, 8, "ogm_gemv_kernel<FmtQ51,gemm>"),
    (96, 40, 20, "ogm_gemv_kernel<FmtQ51,gemm>")])
def test_q5_1_batches_on_the_small_batch_kernel(be, in_dim, out_dim, T, kernel):
    """From nine tokens on (rows of a multiple of 64 inputs) Q5_1 takes the per-32 types' small-batch GEMM, whatever
    the batch (with sixteen waves where the launch has at most 256 workgroups, the rows 64 blocks and the LDS room): a block's term is ad * (dw * dot32 + m * block_sum) (dot_q5_1, vecdot.rs:2886-2899), the block sums of
    the activations from a second matrix instruction against ones; every bit of the CPU path's."""
    raw = synth_weights(Q5_1, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T)
    got = be.matmul(x, T, qm(raw, Q5_1, in_dim, out_dim))
    assert be.last_kernel() == kernel
    assert_bits(got, oracle.matmul(Q5_1, raw, in_dim, out_dim, x, T), "Q5_1 batch")


def test_q5_1_extreme_sums_on_the_small_batch_kernel(be):
    """All weights 31 (and 0) with the largest minimum against activations of +-127."""
    in_dim, out_dim, T = 256, 40, 24
    blocks = np.zeros((out_dim * 8, 24), np.uint8)
    blocks[:, 0:2] = np.frombuffer(np.float16(0.0078125).tobytes(), np.uint8)
    blocks[:, 2:4] = np.frombuffer(np.float16(-3.5).tobytes(), np.uint8)
    blocks[0::2, 4:] = 0xFF
    raw = blocks.reshape(-1)
    x = np.full((T, in_dim), 127.0, np.float32)
    x[1::2] *= -1
    x[:, 5::11] = -127.0
    got = be.matmul(x, T, qm(raw, Q5_1, in_dim, out_dim))
    assert be.last_kernel() == "ogm_gemm_sb_flat_kernel"
    assert_bits(got, oracle.matmul(Q5_1, raw, in_dim, out_dim, x, T), "Q5_1 extreme sums")


@pytest.mark.parametrize("in_dim,out_dim,T,kernel", [
    (256, 5, 9, "ogm_gemm_sb_q2k_kernel"), (1024, 130, 17, "ogm_gemm_sb_q2k_kernel"), (768, 257, 40, "ogm_gemm_sb_q2k_kernel"),
    (2048, 129, 300, "ogm_gemm_sb_q2k_kernel"), (14336, 70, 33, "ogm_gemm_sb_q2k_kernel"),
    (24576, 3, 10, "ogm_gemm_sb_q2k_kernel"), (256, 1, 1000, "ogm_gemm_sb_q2k_kernel"),
    (512, 31, 8, "ogm_gemv_kernel<FmtQ2KGen,gemm>")])
def test_q2_k_batches_on_the_matrix_cores(be, in_dim, out_dim, T, kernel):
    """From nine tokens on Q2_K's several-token arithmetic (unpack_q2_k + dot_unpacked over per-32 activations,
    vecdot.rs:1144-1164, 420-425, 1722-1728: sixteen terms a super-block, added in group order) runs on a kernel whose
    waves take the groups of a super-block, a group one K = 16 int8 matrix instruction and a second one against ones
    for the activations' sum: every bit of the CPU path's."""
    raw = synth_weights(Q2_K, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T)
    got = be.matmul(x, T, qm(raw, Q2_K, in_dim, out_dim))
    assert be.last_kernel() == kernel
    assert_bits(got, oracle.matmul(Q2_K, raw, in_dim, out_dim, x, T), "Q2_K batch")


def test_q2_k_extreme_sums_on_the_matrix_cores(be):
    """All weights 3, scales and minimums 15, against activations of +-127."""
    in_dim, out_dim, T = 1024, 40, 24
    blocks = np.full((out_dim * 4, 84), 0xFF, np.uint8)
    blocks[:, 80:82] = np.frombuffer(np.float16(0.01).tobytes(), np.uint8)
    blocks[:, 82:84] = np.frombuffer(np.float16(0.02).tobytes(), np.uint8)
    blocks[1::2, 16:80] = 0x00
    raw = blocks.reshape(-1)
    x = np.full((T, in_dim), 127.0, np.float32)
    x[1::2] *= -1
    x[:, ::7] = 126.0
    got = be.matmul(x, T, qm(raw, Q2_K, in_dim, out_dim))
    assert be.last_kernel() == "ogm_gemm_sb_q2k_kernel"
    assert_bits(got, oracle.matmul(Q2_K, raw, in_dim, out_dim, x, T), "Q2_K extreme sums")


@pytest.mark.parametrize("chunks", [1, 2])
@pytest.mark.parametrize("t", [Q4_K, Q5_K, Q6_K, Q3_K, IQ4_XS])
@pytest.mark.parametrize("in_dim,out_dim,T", [(256, 5, 9), (1024, 100, 33), (4096, 70, 40), (768, 200, 70), (2304, 33, 128)])
def test_small_batch_kernels_read_rows_or_operand_chunks(be, t, in_dim, out_dim, T, chunks):
    """The K-quants' small-batch kernels take their int8 activations from the token rows or, where the quantizer
    also wrote them, from the 1 KiB operand chunks of 32 tokens x 32 inputs (tokens past the batch's last in a chunk
    are never stored): the same bits either way, on full and ragged token and row tiles (gemm_k_q4_k, gemm_k_q6_k,
    gemm_k_iq4_xs, vecdot.rs:2213-2398)."""
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim + T + t)
    x = synth_x(T, in_dim, seed=T + 3)
    be.set_tuning("gemm_small_max_tokens", 1024)
    be.set_tuning("gemm_act_chunks", chunks)
    try:
        got = be.matmul(x, T, qm(raw, t, in_dim, out_dim))
        assert "ogm_gemm_sb_" in be.last_kernel(), be.last_kernel()
    finally:
        be.set_tuning("gemm_small_max_tokens", 0)
        be.set_tuning("gemm_act_chunks", 0)
    assert_bits(got, oracle.matmul(t, raw, in_dim, out_dim, x, T), f"type {t}, {T} tokens, act_chunks {chunks}")


@pytest.mark.parametrize("t", [Q4_K, Q6_K, IQ4_XS])
@pytest.mark.parametrize("T", [12, 40, 130])
def test_two_step_batches_share_one_quantization(be, t, T):
    """ogm_act_quantize_dev once, then several weights over the same batch (one by one and in one grouped call), as
    arch/mod.rs:1082-1096 does for q, k, v: the bits of Backend::matmul on each.  From 25 tokens the quantize step also
    writes the operand chunks the matrix-core kernels read; the calls that follow must find them, whatever kernel each
    matrix's size sends it to."""
    from orangu_amd import hiprt
    in_dim = 1024
    outs = (70, 300, 33)
    raws = [synth_weights(t, in_dim, o, seed=80 + o + T) for o in outs]
    x = synth_x(T, in_dim, seed=90 + T)
    hs = [be.upload_raw(r, t, in_dim, o) for r, o in zip(raws, outs)]
    xd = hiprt.DeviceBuffer.from_numpy(x)
    yds = [hiprt.DeviceBuffer(4 * T * o) for o in outs]
    try:
        want = [oracle.matmul(t, r, in_dim, o, x, T) for r, o in zip(raws, outs)]
        for yd in yds:
            yd.fill(0xFF)
        hiprt.device_synchronize()   # (the fills run on another stream than the library's)
        be.act_quantize_dev(t, xd.ptr, in_dim, T)
        for h, yd in zip(hs, yds):
            be.matmul_act_dev(h, T, yd.ptr, False)
        hiprt.device_synchronize()
        for yd, w, o in zip(yds, want, outs):
            assert_bits(yd.to_numpy(np.float32, T * o), w, f"two-step, one by one, {o} rows, {be.last_kernel()}")
            yd.fill(0xFF)
        hiprt.device_synchronize()
        be.matmul_multi_act_dev(hs, T, [yd.ptr for yd in yds], False)
        hiprt.device_synchronize()
        for yd, w, o in zip(yds, want, outs):
            assert_bits(yd.to_numpy(np.float32, T * o), w, f"two-step, grouped, {o} rows, {be.last_kernel()}")
    finally:
        for h in hs:
            be.free_weight(h)
        xd.free()
        for yd in yds:
            yd.free()

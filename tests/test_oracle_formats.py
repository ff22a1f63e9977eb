"""Pins the oracle's block formats against what the reference's own tests hold
(engine/quant.rs tests, cited per case).  CPU only."""
import json
import os

import numpy as np
import pytest

import oracle
from helpers import IQ4_NL, Q3_K, Q4_0, Q4_K, Q5_0, Q5_K, Q6_K, Q8_0

# quant.rs:1389-1417 GOLDEN (the types on the path), kept as data in tests/golden/
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "dequantize_checksums.json")) as _f:
    GOLDEN = [(v["ggml_type"], v["name"], v["count"], int(v["checksum"], 16)) for v in json.load(_f)["vectors"]]
assert {g[0] for g in GOLDEN} == {Q4_0, Q5_0, Q8_0, IQ4_NL, Q3_K, Q4_K, Q5_K, Q6_K, 7, 10, 23}   # + Q5_1, Q2_K, IQ4_XS


@pytest.mark.parametrize("ggml_type,name,count,expected", GOLDEN)
def test_dequantizing_every_type_is_unchanged(ggml_type, name, count, expected):
    """quant.rs:1451-1463: bit checksum of dequantize(fixture_bytes).  The Q4_K and Q6_K fixtures
    contain NaN scale fields, so this also pins NaN payload propagation."""
    n = oracle.tensor_byte_size(ggml_type, count)
    data = oracle.fixture_bytes(n)
    values = oracle.dequantize(ggml_type, data, count)
    assert values.size == count
    assert oracle.bit_checksum(values) == expected, name


def test_fixture_bytes_is_xorshift64():
    """Independent restatement of quant.rs:1427-1437 in Python integers."""
    state = 0x2545F4914F6CDD1D
    want = []
    for _ in range(64):
        state ^= (state << 13) & 0xFFFFFFFFFFFFFFFF
        state ^= state >> 7
        state ^= (state << 17) & 0xFFFFFFFFFFFFFFFF
        want.append((state >> 33) & 0xFF)
    assert oracle.fixture_bytes(64).tolist() == want


def test_tensor_byte_size_and_block_layout():
    """quant.rs:132-169, 344-357."""
    assert oracle.tensor_byte_size(Q8_0, 256) == 8 * 34
    assert oracle.tensor_byte_size(Q4_K, 512) == 2 * 144
    assert oracle.tensor_byte_size(Q6_K, 512) == 2 * 210
    assert oracle.tensor_byte_size(Q5_K, 256) == 176  # quant.rs:1701
    assert oracle.tensor_byte_size(Q3_K, 512) == 2 * 110
    assert oracle.tensor_byte_size(Q4_0, 64) == 2 * 18 and oracle.tensor_byte_size(Q5_0, 64) == 2 * 22
    assert oracle.tensor_byte_size(IQ4_NL, 64) == 2 * 18
    assert oracle.tensor_byte_size(Q4_K, 100) == -2  # not a whole number of blocks
    assert oracle.tensor_byte_size(99, 256) == -1  # unknown type


def test_f16_conversion_matches_ieee_for_all_65536_inputs():
    """quant.rs:1671-1690: every finite value, zero, subnormal and infinity equals IEEE binary16
    (numpy's float16 is the independent implementation); a NaN stays a NaN with payload kept."""
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_bits_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    # payload: mantissa shifted left by 13, sign preserved (quant.rs:493-497).  The value comes
    # back through a C float return and a Python float, which quiets a signalling NaN, so the
    # quiet bit is masked on both sides; the golden checksums above pin the payload bits inside
    # dequantize, where no such hop exists.
    quiet = np.uint32(0x00400000)
    gb = got[nan].view(np.uint32) | quiet
    hb = bits[nan].astype(np.uint32)
    assert np.array_equal(gb, ((hb & 0x8000) << 16) | 0x7F800000 | ((hb & 0x3FF) << 13) | quiet)


def _f16(v):
    return np.frombuffer(np.float16(v).tobytes(), np.uint8)


def test_dequantize_q8_0_scales_signed_bytes():
    """quant.rs:1818-1828."""
    qs = np.zeros(32, np.int8)
    qs[0], qs[1] = 1, -1
    block = np.concatenate([_f16(2.0), qs.view(np.uint8)])
    out = oracle.dequantize(Q8_0, block, 32)
    assert out[0] == 2.0 and out[1] == -2.0
    assert np.all(out[2:] == 0.0)


def test_dequantize_q4_k_matches_the_reference_scale_unpacking():
    """quant.rs:1846-1865: scale 1 / min 0 for all eight sub-blocks, nibble 5 -> 5.0."""
    scales = np.array([1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1], np.uint8)
    block = np.concatenate([_f16(1.0), _f16(0.0), scales, np.full(128, 0x55, np.uint8)])
    out = oracle.dequantize(Q4_K, block, 256)
    assert out.size == 256
    assert np.all(np.abs(out - 5.0) < 1e-5)


def test_get_scale_min_k4_against_bit_by_bit_decode():
    """quant.rs:653-662 against ggml's published layout decoded field by field: sub-blocks 0..3
    keep their 6 bits in bytes 0..3 (scale) and 4..7 (min); sub-blocks 4..7 keep the low 4 bits in
    bytes 8..11 (scale low nibble, min high nibble) and the top 2 bits in the top 2 bits of bytes
    0..3 (scale) and 4..7 (min).  A wrong index or shift fails for a random byte pattern."""
    rng = np.random.default_rng(3)
    for _ in range(50):
        b = rng.integers(0, 256, 12, dtype=np.uint8)
        for j in range(8):
            if j < 4:
                sc, m = b[j] % 64, b[j + 4] % 64
            else:
                sc = (b[j + 4] % 16) + 16 * (b[j - 4] // 64)
                m = (b[j + 4] // 16) + 16 * (b[j] // 64)
            assert oracle.get_scale_min_k4(j, b) == (int(sc), int(m))


def test_dequantize_q4_k_sub_block_order_and_min():
    """Distinct scale and min per sub-block, distinct nibbles per half: pins element order
    (low nibbles of qs[32g..] are sub-block 2g, high nibbles 2g+1; quant.rs:679-690) and the
    sign of the min term."""
    sc = [3, 5, 7, 9, 11, 13, 15, 17]
    mn = [1, 2, 3, 4, 21, 22, 23, 24]
    scales = np.zeros(12, np.uint8)
    for j in range(4):
        scales[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        scales[j + 4] = mn[j] | ((mn[j + 4] >> 4) << 6)
        scales[j + 8] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
    qs = np.zeros(128, np.uint8)
    for g in range(4):
        for l in range(32):
            lo, hi = (l + g) % 16, (3 * l + g) % 16
            qs[32 * g + l] = lo | (hi << 4)
    block = np.concatenate([_f16(0.5), _f16(0.25), scales, qs])
    out = oracle.dequantize(Q4_K, block, 256)
    for g in range(4):
        for l in range(32):
            lo, hi = (l + g) % 16, (3 * l + g) % 16
            assert out[64 * g + l] == 0.5 * sc[2 * g] * lo - 0.25 * mn[2 * g]
            assert out[64 * g + 32 + l] == 0.5 * sc[2 * g + 1] * hi - 0.25 * mn[2 * g + 1]


def test_dequantize_q6_k_zero_quant_gives_the_offset_scaled_value():
    """quant.rs:1891-1903."""
    block = np.concatenate([np.zeros(128, np.uint8), np.zeros(64, np.uint8),
                            np.full(16, 2, np.uint8), _f16(1.0)])
    out = oracle.dequantize(Q6_K, block, 256)
    assert np.all(out == -64.0)


def test_dequantize_q6_k_treats_scales_as_signed():
    """quant.rs:1910-1921."""
    block = np.concatenate([np.zeros(128, np.uint8), np.zeros(64, np.uint8),
                            np.full(16, 0xFE, np.uint8), _f16(1.0)])
    out = oracle.dequantize(Q6_K, block, 256)
    assert np.all(out == 64.0)


def test_dequantize_q6_k_element_order():
    """Every element gets its own 6-bit value q = e % 64 and every 16-group its own scale; packs
    them by ggml's published layout (element 128h+32r+l: nibble in ql[64h+32(r&1)+l] low for r<2
    else high, top 2 bits at qh[32h+l] >> 2r, scale 8h+2r+l/16) and expects d*sc*(q-32)."""
    ql = np.zeros(128, np.uint8)
    qh = np.zeros(64, np.uint8)
    sc = np.arange(-8, 8, dtype=np.int8)
    for h in range(2):
        for r in range(4):
            for l in range(32):
                e = 128 * h + 32 * r + l
                q = (e * 7 + 3) % 64
                nib, top = q & 0xF, q >> 4
                idx = 64 * h + 32 * (r & 1) + l
                ql[idx] |= nib if r < 2 else nib << 4
                qh[32 * h + l] |= top << (2 * r)
    block = np.concatenate([ql, qh, sc.view(np.uint8), _f16(0.5)])
    out = oracle.dequantize(Q6_K, block, 256)
    for e in range(256):
        h, r, l = e // 128, (e % 128) // 32, e % 32
        q = (e * 7 + 3) % 64
        assert out[e] == 0.5 * float(sc[8 * h + 2 * r + l // 16]) * (q - 32), e


def test_dequantize_q5_k_applies_the_high_bit_from_qh():
    """quant.rs:1872-1888: d = 1, dmin = 0, every scale 1, every qh bit set, every nibble 0: all
    256 elements are 1 * 1 * (0 + 16) - 0 = 16."""
    block = np.zeros(176, np.uint8)
    block[0:2] = _f16(1.0)
    block[4:16] = [1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]
    block[16:48] = 0xFF
    out = oracle.dequantize(Q5_K, block, 256)
    assert out.size == 256 and np.all(out == 16.0)


def test_dequantize_q5_k_bit_to_sub_block_mapping():
    """Bit j of qh[l] is the fifth bit of element l of sub-block j (quant.rs:703-742): one qh bit
    at a time lights exactly one element; with nibbles set, low nibbles are the even sub-blocks."""
    for j in range(8):
        for l in (0, 13, 31):
            block = np.zeros(176, np.uint8)
            block[0:2] = _f16(1.0)
            block[4:16] = [1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]
            block[16 + l] = 1 << j
            out = oracle.dequantize(Q5_K, block, 256)
            want = np.zeros(256, np.float32)
            want[32 * j + l] = 16.0
            assert np.array_equal(out, want), (j, l)
    block = np.zeros(176, np.uint8)
    block[0:2] = _f16(1.0)
    block[2:4] = _f16(0.5)
    block[4:16] = [1, 2, 3, 4, 1, 1, 1, 1, 0x15, 0x16, 0x17, 0x18]   # sc 1..8, mins 1
    block[48:] = 0x21                                                # low nibble 1, high nibble 2
    out = oracle.dequantize(Q5_K, block, 256).reshape(8, 32)
    for j in range(8):
        nib = 1 if j % 2 == 0 else 2
        assert np.all(out[j] == np.float32(j + 1) * nib - np.float32(0.5)), j


def test_unpack_q3_k_scales_against_bit_by_bit_decode():
    """quant.rs:883-897: low four bits of scales 0..8 in the low nibbles of bytes 0..8, of scales
    8..16 in their high nibbles; the two high bits of scale i at bit 2 * (i / 4) of byte 8 + i % 4.
    Also ggml's kmask shuffle on little-endian words, as a second formulation."""
    rng = np.random.default_rng(3)
    for _ in range(20):
        packed = rng.integers(0, 256, 12, dtype=np.uint8)
        got = oracle.unpack_q3_k_scales(packed)
        want = np.zeros(16, np.int32)
        for i in range(16):
            low = packed[i] & 0xF if i < 8 else packed[i - 8] >> 4
            high = (packed[8 + i % 4] >> (2 * (i // 4))) & 3
            want[i] = int(low) | (int(high) << 4)
        assert np.array_equal(got, want)
        a = [int.from_bytes(packed[4 * k:4 * k + 4].tobytes(), "little") for k in range(3)]
        k1, k2 = 0x03030303, 0x0F0F0F0F
        tmp = a[2]
        w = [(a[0] & k2) | (((tmp >> 0) & k1) << 4), (a[1] & k2) | (((tmp >> 2) & k1) << 4),
             ((a[0] >> 4) & k2) | (((tmp >> 4) & k1) << 4), ((a[1] >> 4) & k2) | (((tmp >> 6) & k1) << 4)]
        ggml = np.frombuffer(b"".join(x.to_bytes(4, "little") for x in w), np.uint8).astype(np.int32)
        assert np.array_equal(got, ggml)


def _q3k_block(hmask=0x00, qs=0x00, scales=0x20, d=1.0):
    block = np.zeros(110, np.uint8)
    block[0:32] = hmask
    block[32:96] = qs
    block[96:108] = scales
    block[108:110] = _f16(d)
    return block


# scale bytes 0x20: low nibbles 0 (scales 0..8), high nibbles 2 (scales 8..16); the byte's bits 4..5
# are also the high bits of scales 8..12: scales = 0 x 8, 34 x 4, 2 x 4, each minus 32
Q3K_SC_0X20 = np.array([0] * 8 + [34] * 4 + [2] * 4, np.float32) - 32


def test_dequantize_q3_k_inverted_high_bit_and_signed_scales():
    """vecdot.rs:3938-3968 on the dequantizer: hmask clear subtracts 4, hmask set subtracts nothing;
    the six-bit scales are biased by 32 (quant.rs:857)."""
    per_elem = np.repeat(Q3K_SC_0X20, 16)
    assert np.array_equal(oracle.dequantize(Q3_K, _q3k_block(hmask=0x00), 256), per_elem * -4)
    assert np.all(oracle.dequantize(Q3_K, _q3k_block(hmask=0xFF), 256) == 0.0)
    assert np.array_equal(oracle.dequantize(Q3_K, _q3k_block(hmask=0xFF, qs=0xFF), 256), per_elem * 3)


def test_dequantize_q3_k_element_order():
    """Run p (32 elements) takes qs[32 (p / 4) ..][j] >> 2 (p % 4) and hmask bit p; groups of 16
    take scales 2p and 2p + 1 (quant.rs:851-868).  One qs bit, one hmask bit at a time."""
    for p in range(8):
        for j in (0, 15, 16, 31):
            g = 2 * p + j // 16
            block = _q3k_block(hmask=0xFF)
            block[32 + 32 * (p // 4) + j] = 1 << (2 * (p % 4))
            want = np.zeros(256, np.float32)
            want[32 * p + j] = Q3K_SC_0X20[g] * 1
            assert np.array_equal(oracle.dequantize(Q3_K, block, 256), want), (p, j)
            block = _q3k_block(hmask=0xFF)
            block[j] = 0xFF ^ (1 << p)          # clear hmask bit p of element j only
            want = np.zeros(256, np.float32)
            want[32 * p + j] = Q3K_SC_0X20[g] * -4
            assert np.array_equal(oracle.dequantize(Q3_K, block, 256), want), (p, j)


KVALUES_IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)


def test_dequantize_q4_0_and_q5_0_apply_their_fixed_offsets():
    """quant.rs:1768-1775, 1807-1815: all-zero quants at d = 1 are -8 (Q4_0) and -16 (Q5_0)."""
    block = np.zeros(18, np.uint8)
    block[0:2] = _f16(1.0)
    assert np.all(oracle.dequantize(Q4_0, block, 32) == -8.0)
    block = np.zeros(22, np.uint8)
    block[0:2] = _f16(1.0)
    assert np.all(oracle.dequantize(Q5_0, block, 32) == -16.0)


def test_dequantize_iq4_nl_uses_the_codebook_not_a_linear_offset():
    """quant.rs:1785-1803: zero nibbles are level 0 = -127 (a linear Q4_0 decode would say -8);
    byte j = j | j << 4 gives the sixteen levels in order in both halves."""
    block = np.zeros(18, np.uint8)
    block[0:2] = _f16(1.0)
    assert np.all(oracle.dequantize(IQ4_NL, block, 32) == -127.0)
    block[2:] = [j | (j << 4) for j in range(16)]
    out = oracle.dequantize(IQ4_NL, block, 32)
    assert np.array_equal(out[:16], KVALUES_IQ4NL) and np.array_equal(out[16:], KVALUES_IQ4NL)


def test_per_32_nibble_types_element_order_and_fifth_bit():
    """Element j < 16 is the low nibble of qs[j], element 16 + j the high nibble (quant.rs:546-551);
    Q5_0's fifth bit of element e is bit e of the little-endian qh (quant.rs:571-574)."""
    rng = np.random.default_rng(5)
    for _ in range(10):
        qs = rng.integers(0, 256, 16, dtype=np.uint8)
        qh = rng.integers(0, 256, 4, dtype=np.uint8)
        nib = np.concatenate([qs & 15, qs >> 4]).astype(np.int64)
        b4 = np.concatenate([_f16(1.0), qs])
        assert np.array_equal(oracle.dequantize(Q4_0, b4, 32), (nib - 8).astype(np.float32))
        assert np.array_equal(oracle.dequantize(IQ4_NL, b4, 32), KVALUES_IQ4NL[nib])
        bits = np.unpackbits(qh, bitorder="little").astype(np.int64)
        b5 = np.concatenate([_f16(1.0), qh, qs])
        assert np.array_equal(oracle.dequantize(Q5_0, b5, 32), (nib + 16 * bits - 16).astype(np.float32))

"""CPU-side checks of the product library: it loads, exports every symbol the header declares,
and its host-only functions (predicates, repack and inverse) behave.  No GPU compute here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from helpers import BLOCK, IQ4_NL, IQ4_XS, Q2_K, Q3_K, Q4_0, Q4_K, Q5_0, Q5_1, Q5_K, Q6_K, Q8_0, row_bytes
from orangu_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return capi.load_library()


def test_library_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "orangu_mi355x.h")).read()
    declared = set(re.findall(r"\b(ogm_[a-z0-9_]+)\s*\(", header))
    declared -= {"ogm_op", "ogm_ctx", "ogm_weight", "ogm_status"}
    assert declared, "no declarations found"
    missing = [s for s in sorted(declared) if not hasattr(lib, s)]
    assert not missing, missing
    assert declared == set(capi.SYMBOLS), declared ^ set(capi.SYMBOLS)


def test_supports_predicates_follow_vecdot(lib):
    """vecdot.rs:274-283 for the types built; Backend::supports_type (mod.rs:493)."""
    assert lib.ogm_supports_type(Q8_0) and lib.ogm_supports_type(Q4_K) and lib.ogm_supports_type(Q6_K)
    assert lib.ogm_supports_type(13) and lib.ogm_supports(13, 256) and not lib.ogm_supports(13, 128)   # Q5_K
    assert lib.ogm_supports_type(11) and lib.ogm_supports(11, 512) and not lib.ogm_supports(11, 896)   # Q3_K
    for t in (2, 6, 20):   # Q4_0, Q5_0, IQ4_NL
        assert lib.ogm_supports_type(t) and lib.ogm_supports(t, 896) and not lib.ogm_supports(t, 24)
    assert lib.ogm_supports_type(Q5_1) and lib.ogm_supports(Q5_1, 896) and not lib.ogm_supports(Q5_1, 24)
    for t in (Q2_K, IQ4_XS):
        assert lib.ogm_supports_type(t) and lib.ogm_supports(t, 2048) and not lib.ogm_supports(t, 896)
    assert not lib.ogm_supports_type(0) and not lib.ogm_supports_type(3) and not lib.ogm_supports_type(16)
    assert lib.ogm_supports(Q8_0, 96) and not lib.ogm_supports(Q8_0, 100)
    assert lib.ogm_supports(Q4_K, 512) and not lib.ogm_supports(Q4_K, 896)
    assert lib.ogm_supports(Q6_K, 256) and not lib.ogm_supports(Q6_K, 0)
    for t, (bb, be) in BLOCK.items():
        a, b = C.c_uint32(), C.c_uint32()
        assert lib.ogm_block_layout(t, C.byref(a), C.byref(b)) == 0
        assert (a.value, b.value) == (bb, be)
    assert lib.ogm_block_layout(3, None, None) == -2   # Q4_1: not built


def tiling(upr, out_dim):
    """ogm_layout.h: tiles of R rows x C blocks, C = 4 / 2 / 1 by divisibility of blocks per row."""
    C_ = 4 if upr % 4 == 0 else (2 if upr % 2 == 0 else 1)
    R = 64 // C_
    return C_, R, upr // C_, (out_dim + R - 1) // R


# bytes a unit takes in the tile-planar form: the raw block, except Q3_K and IQ4_XS whose last piece is padded
TILE_UNIT = {Q4_0: 18, Q5_0: 22, Q5_1: 24, Q8_0: 34, IQ4_NL: 18, Q2_K: 84, Q3_K: 112, Q4_K: 144, Q5_K: 176, Q6_K: 210,
             IQ4_XS: 144}


@pytest.mark.parametrize("ggml_type", [Q8_0, Q5_0, Q4_0, IQ4_NL, Q3_K, Q4_K, Q5_K, Q6_K, Q5_1, Q2_K, IQ4_XS])
@pytest.mark.parametrize("in_blocks,out_dim", [(1, 1), (3, 11), (16, 64), (7, 130), (6, 33), (8, 70)])
def test_repack_is_a_bijection_on_the_raw_bytes(lib, ggml_type, in_blocks, out_dim):
    bb, be = BLOCK[ggml_type]
    in_dim = in_blocks * be
    rb = row_bytes(ggml_type, in_dim)
    rng = np.random.default_rng(in_blocks * 1000 + out_dim)
    raw = rng.integers(0, 256, rb * out_dim, dtype=np.uint8)
    size = lib.ogm_repacked_size(ggml_type, in_dim, out_dim)
    C_, R, nct, nrb = tiling(in_blocks, out_dim)
    assert size == nrb * nct * 64 * TILE_UNIT[ggml_type]
    packed = np.full(size, 0xAA, np.uint8)
    assert lib.ogm_repack_host(ggml_type, raw.ctypes.data, rb, in_dim, out_dim, packed.ctypes.data) == 0
    back = np.zeros_like(raw)
    assert lib.ogm_unrepack_host(ggml_type, packed.ctypes.data, rb, in_dim, out_dim, back.ctypes.data) == 0
    assert np.array_equal(back, raw)
    if out_dim % R == 0 and TILE_UNIT[ggml_type] == bb:
        # no padding rows or bytes: the packed form is a permutation of the raw bytes
        assert np.array_equal(np.bincount(packed, minlength=256), np.bincount(raw, minlength=256))


@pytest.mark.parametrize("t,npieces,piece_off,tail_off,tail", [(Q4_K, 9, 0, 0, 0), (Q6_K, 13, 0, 208, 2),
                                                              (Q8_0, 2, 2, 0, 2), (Q5_K, 11, 0, 0, 0),
                                                              (Q3_K, 7, 0, 0, 0), (Q4_0, 1, 2, 0, 2),
                                                              (Q5_0, 1, 6, 0, 6), (IQ4_NL, 1, 2, 0, 2),
                                                              (Q5_1, 1, 8, 0, 8), (Q2_K, 5, 0, 80, 4), (IQ4_XS, 9, 0, 0, 0)])
@pytest.mark.parametrize("in_blocks,out_dim", [(8, 70), (6, 40), (3, 65)])
def test_repack_places_pieces_in_planes(lib, t, npieces, piece_off, tail_off, tail, in_blocks, out_dim):
    """Unit (row o, block b): tile (o / R) * nct + b / C, lane (b % C) * R + o % R; piece p at
    tile * tile bytes + p * 1024 + lane * 16, tails after the pieces; padding rows zero, and so
    are the two bytes that complete Q3_K's last piece."""
    bb, be = BLOCK[t]
    in_dim = in_blocks * be
    rb = row_bytes(t, in_dim)
    raw = ((np.arange(rb * out_dim, dtype=np.uint64) * 2654435761) >> 7).astype(np.uint8)
    C_, R, nct, nrb = tiling(in_blocks, out_dim)
    packed = np.full(lib.ogm_repacked_size(t, in_dim, out_dim), 0x5A, np.uint8)
    assert lib.ogm_repack_host(t, raw.ctypes.data, rb, in_dim, out_dim, packed.ctypes.data) == 0
    seen = np.zeros(packed.size, bool)
    for o in range(out_dim):
        for b in range(in_blocks):
            base = ((o // R) * nct + b // C_) * 64 * TILE_UNIT[t]
            lane = (b % C_) * R + o % R
            src = o * rb + b * bb
            for p in range(npieces):
                off = base + p * 1024 + lane * 16
                have = min(16, bb - piece_off - p * 16)
                assert np.array_equal(packed[off:off + have], raw[src + piece_off + p * 16:src + piece_off + p * 16 + have])
                seen[off:off + have] = True
            if tail:
                off = base + npieces * 1024 + lane * tail
                assert np.array_equal(packed[off:off + tail], raw[src + tail_off:src + tail_off + tail])
                seen[off:off + tail] = True
    assert not packed[~seen].any()  # rows that pad the last row block are zero units


def test_repack_rejects_bad_shapes(lib):
    buf = np.zeros(4096, np.uint8)
    assert lib.ogm_repack_host(3, buf.ctypes.data, 20, 32, 1, buf.ctypes.data) == -2  # Q4_1: no kernel
    assert lib.ogm_repack_host(Q4_K, buf.ctypes.data, 144, 128, 1, buf.ctypes.data) == -2  # in_dim % 256
    assert lib.ogm_repack_host(Q4_K, buf.ctypes.data, 100, 256, 1, buf.ctypes.data) == -1  # row_bytes
    assert lib.ogm_repack_host(Q4_K, None, 144, 256, 1, buf.ctypes.data) == -1
    assert lib.ogm_repack_host(Q4_K, buf.ctypes.data, 144, 256, 0, buf.ctypes.data) == -1
    assert lib.ogm_repacked_size(Q4_K, 100, 4) == 0


def test_init_without_a_device_is_a_status_not_a_crash(lib):
    """RocmBackend::try_init never panics (rocm.rs:168-173).  Only meaningful without a GPU."""
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    ctx = C.c_void_p()
    rc = lib.ogm_init(0, C.byref(ctx))
    assert rc == -3 and not ctx.value
    assert b"device" in lib.ogm_last_error(None).lower()
    from orangu_amd import Mi355xBackend
    assert Mi355xBackend.try_init() is None
    # null-context calls return a status
    assert lib.ogm_matmul(None, None, None, 1, None) == -1
    assert lib.ogm_set_tuning(None, b"gemv_wg_waves", 1) == -1


def test_every_tuning_key_the_library_accepts_is_documented_in_the_header():
    """ogm_set_tuning's keys are compared by name in ogm_api.cpp; the header is where a host maintainer
    reads what each one does."""
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = open(os.path.join(root, "orangu_amd", "csrc", "ogm_api.cpp")).read()
    header = open(os.path.join(root, "include", "orangu_mi355x.h")).read()
    keys = re.findall(r'strcmp\(key, "([a-z0-9_]+)"\)', src)
    assert len(keys) >= 10 and len(set(keys)) == len(keys)
    missing = [k for k in keys if f'"{k}"' not in header]
    assert not missing, missing

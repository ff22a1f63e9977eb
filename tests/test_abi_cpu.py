"""CPU-side checks of the product library: it loads, exports every symbol the header declares,
and its host-only functions (predicates, repack and inverse) behave.  No GPU compute here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from helpers import BLOCK, Q4_K, Q6_K, Q8_0, row_bytes
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
    """vecdot.rs:274-283 for the three types; Backend::supports_type (mod.rs:493)."""
    assert lib.ogm_supports_type(Q8_0) and lib.ogm_supports_type(Q4_K) and lib.ogm_supports_type(Q6_K)
    assert not lib.ogm_supports_type(0) and not lib.ogm_supports_type(13)
    assert lib.ogm_supports(Q8_0, 96) and not lib.ogm_supports(Q8_0, 100)
    assert lib.ogm_supports(Q4_K, 512) and not lib.ogm_supports(Q4_K, 896)
    assert lib.ogm_supports(Q6_K, 256) and not lib.ogm_supports(Q6_K, 0)
    for t, (bb, be) in BLOCK.items():
        a, b = C.c_uint32(), C.c_uint32()
        assert lib.ogm_block_layout(t, C.byref(a), C.byref(b)) == 0
        assert (a.value, b.value) == (bb, be)
    assert lib.ogm_block_layout(2, None, None) == -2


@pytest.mark.parametrize("ggml_type", [Q8_0, Q4_K, Q6_K])
@pytest.mark.parametrize("in_blocks,out_dim", [(1, 1), (3, 11), (16, 64), (7, 130)])
def test_repack_is_a_bijection_on_the_raw_bytes(lib, ggml_type, in_blocks, out_dim):
    bb, be = BLOCK[ggml_type]
    in_dim = in_blocks * be
    rb = row_bytes(ggml_type, in_dim)
    rng = np.random.default_rng(in_blocks * 1000 + out_dim)
    raw = rng.integers(0, 256, rb * out_dim, dtype=np.uint8)
    size = lib.ogm_repacked_size(ggml_type, in_dim, out_dim)
    units = in_blocks * out_dim
    assert size == (units + 63) // 64 * 64 * bb
    packed = np.full(size, 0xAA, np.uint8)
    assert lib.ogm_repack_host(ggml_type, raw.ctypes.data, rb, in_dim, out_dim, packed.ctypes.data) == 0
    back = np.zeros_like(raw)
    assert lib.ogm_unrepack_host(ggml_type, packed.ctypes.data, rb, in_dim, out_dim, back.ctypes.data) == 0
    assert np.array_equal(back, raw)
    # same multiset of bytes plus zero padding: nothing altered, nothing dropped
    assert np.array_equal(np.bincount(packed, minlength=256) - np.bincount(raw, minlength=256),
                          np.eye(1, 256, 0, dtype=np.int64)[0] * (size - raw.size))


def test_repack_places_pieces_in_planes(lib):
    """Unit u of a Q4_K matrix: piece p at tile*9216 + p*1024 + (u%64)*16."""
    in_dim, out_dim = 512, 70  # 140 units: 2 full tiles + 12
    rb = row_bytes(Q4_K, in_dim)
    raw = np.arange(rb * out_dim, dtype=np.uint32).astype(np.uint8)
    raw = (np.arange(rb * out_dim) * 2654435761 >> 7).astype(np.uint8)
    packed = np.zeros(lib.ogm_repacked_size(Q4_K, in_dim, out_dim), np.uint8)
    lib.ogm_repack_host(Q4_K, raw.ctypes.data, rb, in_dim, out_dim, packed.ctypes.data)
    for u in (0, 1, 63, 64, 100, 139):
        for p in range(9):
            off = (u // 64) * 9216 + p * 1024 + (u % 64) * 16
            assert np.array_equal(packed[off:off + 16], raw[u * 144 + p * 16:u * 144 + p * 16 + 16])
    # Q6_K tail (d) and Q8_0 tail (d) land after the planes
    for t, npieces, tail_off, piece_off in ((Q6_K, 13, 208, 0), (Q8_0, 2, 0, 2)):
        bb, be = BLOCK[t]
        in_dim, out_dim = be * 5, 33
        rb = row_bytes(t, in_dim)
        raw = (np.arange(rb * out_dim) * 40503 >> 5).astype(np.uint8)
        packed = np.zeros(lib.ogm_repacked_size(t, in_dim, out_dim), np.uint8)
        lib.ogm_repack_host(t, raw.ctypes.data, rb, in_dim, out_dim, packed.ctypes.data)
        for u in (0, 63, 64, 164):
            base = (u // 64) * 64 * bb
            for p in range(npieces):
                off = base + p * 1024 + (u % 64) * 16
                src = u * bb + piece_off + p * 16
                assert np.array_equal(packed[off:off + 16], raw[src:src + 16])
            off = base + npieces * 1024 + (u % 64) * 2
            assert np.array_equal(packed[off:off + 2], raw[u * bb + tail_off:u * bb + tail_off + 2])


def test_repack_rejects_bad_shapes(lib):
    buf = np.zeros(4096, np.uint8)
    assert lib.ogm_repack_host(2, buf.ctypes.data, 18, 32, 1, buf.ctypes.data) == -2  # Q4_0: no kernel
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

"""ctypes loader for the CPU oracle (``liborangu_oracle.so``).

TEST INFRASTRUCTURE ONLY.  Tests, the smoke check and the benchmark's ``cpu_baseline`` leg may
import this; the shipped package ``orangu_amd`` never does.  The library is a C restatement of
orangu-server's ``engine::vecdot`` / ``engine::quant`` / ``CpuBackend`` (see
``orangu_oracle.h`` for the per-function citations).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liborangu_oracle.so")

Q4_0, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 2, 6, 7, 8, 10, 11, 12, 13, 14, 20, 23
BLOCK_LAYOUT = {Q4_0: (18, 32), Q5_0: (22, 32), Q5_1: (24, 32), Q8_0: (34, 32), Q2_K: (84, 256), Q3_K: (110, 256),
                Q4_K: (144, 256), Q5_K: (176, 256), Q6_K: (210, 256), IQ4_NL: (18, 32), IQ4_XS: (136, 256)}


def build() -> str:
    """Compile the oracle in place (``make -C oracle``)."""
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        u8p, i8p, f32p, i32p, i16p = (C.c_void_p,) * 5
        sz = C.c_size_t
        L.ogo_f16_bits_to_f32.restype = C.c_float
        L.ogo_f16_bits_to_f32.argtypes = [C.c_uint16]
        L.ogo_get_scale_min_k4.argtypes = [C.c_int, u8p, u8p, u8p]
        L.ogo_block_layout.argtypes = [C.c_uint32, C.POINTER(sz), C.POINTER(sz)]
        L.ogo_tensor_byte_size.restype = C.c_int64
        L.ogo_tensor_byte_size.argtypes = [C.c_uint32, C.c_uint64]
        L.ogo_dequantize.argtypes = [C.c_uint32, u8p, sz, f32p]
        L.ogo_fixture_bytes.argtypes = [sz, u8p]
        L.ogo_bit_checksum.restype = C.c_uint64
        L.ogo_bit_checksum.argtypes = [f32p, sz]
        L.ogo_pseudo_bytes.argtypes = [sz, C.c_uint32, u8p]
        L.ogo_quantize_act.argtypes = [f32p, sz, i8p, f32p, i32p]
        L.ogo_quantize_act_k_row.argtypes = [f32p, sz, i8p, f32p, i32p]
        L.ogo_act_q8k_quantize.argtypes = [f32p, sz, sz, i8p, f32p, i16p]
        L.ogo_act_q8flat_quantize.argtypes = [f32p, sz, sz, i8p, f32p]
        for name in ("ogo_dot16_scalar", "ogo_dot16", "ogo_dot32"):
            getattr(L, name).restype = C.c_int32
            getattr(L, name).argtypes = [i8p, i8p]
        L.ogo_isa_name.restype = C.c_char_p
        L.ogo_force_scalar.argtypes = [C.c_int]
        L.ogo_dot_q8_0.restype = C.c_float
        L.ogo_dot_q8_0.argtypes = [u8p, sz, i8p, f32p]
        L.ogo_dot_q4_k.restype = C.c_float
        L.ogo_dot_q4_k.argtypes = [u8p, sz, i8p, f32p, i32p]
        L.ogo_dot_q6_k.restype = C.c_float
        L.ogo_dot_q6_k.argtypes = [u8p, sz, i8p, f32p]
        L.ogo_dot_k_row_q4_k.restype = C.c_float
        L.ogo_dot_k_row_q4_k.argtypes = [u8p, sz, i8p, f32p, i32p, i32p, i32p]
        L.ogo_dot_k_row_q5_k.restype = C.c_float
        L.ogo_dot_k_row_q5_k.argtypes = [u8p, sz, i8p, f32p, i32p, i32p, i32p]
        L.ogo_dot_k_row_q6_k.restype = C.c_float
        L.ogo_dot_k_row_q6_k.argtypes = [u8p, sz, i8p, f32p, i32p]
        L.ogo_dot_k_row_q3_k.restype = C.c_float
        L.ogo_dot_k_row_q3_k.argtypes = [u8p, sz, i8p, f32p, i32p]
        L.ogo_dot_q5_1.restype = C.c_float
        L.ogo_dot_q5_1.argtypes = [u8p, sz, i8p, f32p, i32p, i32p]
        L.ogo_dot_k_row_iq4_xs.restype = C.c_float
        L.ogo_dot_k_row_iq4_xs.argtypes = [u8p, sz, i8p, f32p, i32p]
        L.ogo_dot_k_row_q2_k.restype = C.c_float
        L.ogo_dot_k_row_q2_k.argtypes = [u8p, sz, i8p, f32p, i32p, i32p, i32p]
        L.ogo_dot_unpacked_q2_k.restype = C.c_float
        L.ogo_dot_unpacked_q2_k.argtypes = [u8p, sz, i8p, f32p, i32p]
        L.ogo_unpack_q3_k_scales.argtypes = [u8p, i32p]
        L.ogo_dot_flat32.restype = C.c_float
        L.ogo_dot_flat32.argtypes = [C.c_uint32, u8p, sz, i8p, f32p, i32p]
        L.ogo_unpack_flat_block.restype = C.c_float
        L.ogo_unpack_flat_block.argtypes = [C.c_uint32, u8p, i8p]
        L.ogo_block_sums_q8_0.argtypes = [u8p, sz, i8p, i32p]
        for name in ("ogo_supports", "ogo_supports_k", "ogo_supports_k_row", "ogo_supports_flat"):
            getattr(L, name).argtypes = [C.c_uint32, sz]
        mm = [C.c_uint32, u8p, sz, sz, sz, f32p, sz, f32p, C.c_int]
        L.ogo_matmul.argtypes = mm
        L.ogo_matmul_decode.argtypes = mm
        L.ogo_matmul_dequant.argtypes = mm
        L.ogo_gemv_act.argtypes = [C.c_uint32, u8p, sz, sz, sz, i8p, f32p, i32p, f32p, C.c_int]
        L.ogo_k_gemm_t.argtypes = [C.c_uint32, u8p, sz, sz, sz, f32p, sz, f32p]
        L.ogo_block_sums.argtypes = [C.c_uint32, u8p, sz, sz, sz, f32p, sz, i32p, i32p]
        _lib = L
    return _lib


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(np.frombuffer(bytes(a), dtype=np.uint8) if isinstance(a, (bytes, bytearray)) else a, dtype=np.uint8)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


# ---------------------------------------------------------------- formats / fixtures

def f16_bits_to_f32(bits: int) -> np.float32:
    return np.float32(lib().ogo_f16_bits_to_f32(bits))


def get_scale_min_k4(j: int, scales) -> tuple[int, int]:
    s = _u8(scales)
    sc, m = np.zeros(1, np.uint8), np.zeros(1, np.uint8)
    lib().ogo_get_scale_min_k4(j, _p(s), _p(sc), _p(m))
    return int(sc[0]), int(m[0])


def tensor_byte_size(ggml_type: int, n: int) -> int:
    return int(lib().ogo_tensor_byte_size(ggml_type, n))


def dequantize(ggml_type: int, data, n: int) -> np.ndarray:
    b = _u8(data)
    out = np.empty(n, np.float32)
    rc = lib().ogo_dequantize(ggml_type, _p(b), n, _p(out))
    if rc != 0:
        raise ValueError(f"ogo_dequantize rc={rc}")
    return out


def fixture_bytes(n: int) -> np.ndarray:
    out = np.empty(n, np.uint8)
    lib().ogo_fixture_bytes(n, _p(out))
    return out


def bit_checksum(values) -> int:
    v = _f32(values)
    return int(lib().ogo_bit_checksum(_p(v), v.size))


def pseudo_bytes(n: int, seed: int) -> np.ndarray:
    out = np.empty(n, np.uint8)
    lib().ogo_pseudo_bytes(n, seed & 0xFFFFFFFF, _p(out))
    return out


# ---------------------------------------------------------------- quantizers

def quantize_act(x):
    """Per-32 scale (vecdot.rs:95-126) -> (q int8[n], d f32[n/32], sums i32[n/16])."""
    x = _f32(x)
    n = x.size
    q, d, s = np.empty(n, np.int8), np.empty(n // 32, np.float32), np.empty(n // 16, np.int32)
    lib().ogo_quantize_act(_p(x), n, _p(q), _p(d), _p(s))
    return q, d, s


def quantize_act_k_row(x):
    """Per-256 scale (vecdot.rs:3030-3053) -> (q int8[n], d f32[n/256], sums i32[n/16])."""
    x = _f32(x)
    n = x.size
    q, d, s = np.empty(n, np.int8), np.empty(n // 256, np.float32), np.empty(n // 16, np.int32)
    lib().ogo_quantize_act_k_row(_p(x), n, _p(q), _p(d), _p(s))
    return q, d, s


def act_q8k_quantize(x, in_dim: int, n_tokens: int):
    """ActQ8K (vecdot.rs:1858-1910) -> q[tile][n/32][4][32], d[tile][n/256][4], bsum[tile][n/256][4][8]."""
    x = _f32(x)
    nt = (n_tokens + 3) // 4
    q = np.zeros((nt, in_dim // 32, 4, 32), np.int8)
    d = np.zeros((nt, in_dim // 256, 4), np.float32)
    b = np.zeros((nt, in_dim // 256, 4, 8), np.int16)
    lib().ogo_act_q8k_quantize(_p(x), in_dim, n_tokens, _p(q), _p(d), _p(b))
    return q, d, b


def act_q8flat_quantize(x, in_dim: int, n_tokens: int):
    x = _f32(x)
    nt = (n_tokens + 3) // 4
    q = np.zeros((nt, in_dim // 32, 4, 32), np.int8)
    d = np.zeros((nt, in_dim // 32, 4), np.float32)
    lib().ogo_act_q8flat_quantize(_p(x), in_dim, n_tokens, _p(q), _p(d))
    return q, d


# ---------------------------------------------------------------- dots

def dot16_scalar(w, x) -> int:
    w, x = np.ascontiguousarray(w, np.int8), np.ascontiguousarray(x, np.int8)
    return int(lib().ogo_dot16_scalar(_p(w), _p(x)))


def dot16(w, x) -> int:
    w, x = np.ascontiguousarray(w, np.int8), np.ascontiguousarray(x, np.int8)
    return int(lib().ogo_dot16(_p(w), _p(x)))


def dot32(w, x) -> int:
    w, x = np.ascontiguousarray(w, np.int8), np.ascontiguousarray(x, np.int8)
    return int(lib().ogo_dot32(_p(w), _p(x)))


def isa_name() -> str:
    return lib().ogo_isa_name().decode()


def force_scalar(on: bool) -> None:
    lib().ogo_force_scalar(1 if on else 0)


def dot_row(ggml_type: int, row, act) -> np.float32:
    """vecdot.rs:2650 dot_row over a per-32 ActQ8 ``(q, d, sums)``."""
    r = _u8(row)
    q, d, s = act
    n = q.size
    L = lib()
    if ggml_type == Q8_0:
        return np.float32(L.ogo_dot_q8_0(_p(r), n, _p(q), _p(d)))
    if ggml_type in (Q4_0, Q5_0, IQ4_NL):
        return np.float32(L.ogo_dot_flat32(ggml_type, _p(r), n, _p(q), _p(d), None))
    if ggml_type == Q4_K:
        return np.float32(L.ogo_dot_q4_k(_p(r), n, _p(q), _p(d), _p(s)))
    if ggml_type == Q6_K:
        return np.float32(L.ogo_dot_q6_k(_p(r), n, _p(q), _p(d)))
    if ggml_type == Q5_1:
        return np.float32(L.ogo_dot_q5_1(_p(r), n, _p(q), _p(d), _p(s), None))
    raise ValueError(ggml_type)


def dot_unpacked_q2_k(row, act) -> np.float32:
    """unpack_q2_k + dot_unpacked (vecdot.rs:1144-1164, 407-428) over a per-32 ActQ8 ``(q, d, sums)``: what
    matmul computes per token for Q2_K at n_tokens > 1."""
    r = _u8(row)
    q, d, s = act
    return np.float32(lib().ogo_dot_unpacked_q2_k(_p(r), q.size, _p(q), _p(d), _p(s)))


def unpack_flat_block(ggml_type: int, block):
    """One block of a symmetric per-32 type as (dw, int8[32]) (vecdot.rs:913-1039)."""
    b = _u8(block)
    w = np.zeros(32, np.int8)
    dw = lib().ogo_unpack_flat_block(ggml_type, _p(b), _p(w))
    return np.float32(dw), w


def unpack_q3_k_scales(packed) -> np.ndarray:
    """quant.rs:883-897."""
    p = _u8(packed)
    out = np.zeros(16, np.int32)
    lib().ogo_unpack_q3_k_scales(_p(p), _p(out))
    return out


def dot_k_row(ggml_type: int, row, act, want_sums: bool = False):
    """vecdot.rs:3103 dot_k_row over a per-256 ActQ8KRow ``(q, d, sums)``."""
    r = _u8(row)
    q, d, s = act
    n = q.size
    isum = np.zeros(n // 256, np.int32)
    imin = np.zeros(n // 256, np.int32)
    L = lib()
    if ggml_type == Q4_K:
        v = L.ogo_dot_k_row_q4_k(_p(r), n, _p(q), _p(d), _p(s), _p(isum), _p(imin))
    elif ggml_type == Q5_K:
        v = L.ogo_dot_k_row_q5_k(_p(r), n, _p(q), _p(d), _p(s), _p(isum), _p(imin))
    elif ggml_type == Q6_K:
        v = L.ogo_dot_k_row_q6_k(_p(r), n, _p(q), _p(d), _p(isum))
    elif ggml_type == Q3_K:
        v = L.ogo_dot_k_row_q3_k(_p(r), n, _p(q), _p(d), _p(isum))
    elif ggml_type == IQ4_XS:
        v = L.ogo_dot_k_row_iq4_xs(_p(r), n, _p(q), _p(d), _p(isum))
    elif ggml_type == Q2_K:
        v = L.ogo_dot_k_row_q2_k(_p(r), n, _p(q), _p(d), _p(s), _p(isum), _p(imin))
    else:
        raise ValueError(ggml_type)
    return (np.float32(v), isum, imin) if want_sums else np.float32(v)


# ---------------------------------------------------------------- CpuBackend

def supports(t, n):
    return bool(lib().ogo_supports(t, n))


def supports_k(t, n):
    return bool(lib().ogo_supports_k(t, n))


def supports_k_row(t, n):
    return bool(lib().ogo_supports_k_row(t, n))


def supports_flat(t, n):
    return bool(lib().ogo_supports_flat(t, n))


def _mm(fn, ggml_type, raw, in_dim, out_dim, x, n_tokens, threads):
    raw = _u8(raw)
    x = _f32(x)
    bb, be = BLOCK_LAYOUT[ggml_type]
    row_bytes = in_dim // be * bb
    assert raw.size == row_bytes * out_dim, (raw.size, row_bytes, out_dim)
    assert x.size == n_tokens * in_dim
    y = np.empty((n_tokens, out_dim), np.float32)
    rc = fn(ggml_type, _p(raw), row_bytes, in_dim, out_dim, _p(x), n_tokens, _p(y), threads)
    if rc != 0:
        raise ValueError(f"oracle matmul rc={rc}")
    return y


def matmul(ggml_type, raw, in_dim, out_dim, x, n_tokens=1, threads=0) -> np.ndarray:
    """CpuBackend::matmul (backend/cpu.rs:445-458): y[n_tokens][out_dim]."""
    return _mm(lib().ogo_matmul, ggml_type, raw, in_dim, out_dim, x, n_tokens, threads)


def gemv_act(ggml_type, raw, in_dim, out_dim, q, d, threads=0) -> np.ndarray:
    """The single-token GEMV of CpuBackend::matmul over an activation that is already quantized:
    q int8 [in_dim], d f32 [in_dim / 32] (per-32 types) or [in_dim / 256] (K-quants); the per-16 sums
    are those of q (vecdot.rs:119-124).  Same dot_row / dot_k_row calls as `matmul` at one token."""
    raw = _u8(raw)
    bb, be = BLOCK_LAYOUT[ggml_type]
    row_bytes = in_dim // be * bb
    assert raw.size == row_bytes * out_dim, (raw.size, row_bytes, out_dim)
    q = np.ascontiguousarray(q, np.int8).reshape(-1)
    d = np.ascontiguousarray(d, np.float32).reshape(-1)
    assert q.size == in_dim and d.size == in_dim // (32 if be == 32 else 256), (q.size, d.size)
    sums = np.ascontiguousarray(q.astype(np.int32).reshape(-1, 16).sum(axis=1), np.int32)
    y = np.empty(out_dim, np.float32)
    rc = lib().ogo_gemv_act(ggml_type, _p(raw), row_bytes, in_dim, out_dim, _p(q), _p(d), _p(sums), _p(y), threads)
    if rc != 0:
        raise ValueError(f"oracle gemv_act rc={rc}")
    return y


def matmul_decode(ggml_type, raw, in_dim, out_dim, x, n_tokens=1, threads=0) -> np.ndarray:
    """CpuBackend::matmul_decode (backend/cpu.rs:466-480)."""
    return _mm(lib().ogo_matmul_decode, ggml_type, raw, in_dim, out_dim, x, n_tokens, threads)


def matmul_dequant(ggml_type, raw, in_dim, out_dim, x, n_tokens=1, threads=0) -> np.ndarray:
    """CpuBackend::matmul_dequant (backend/cpu.rs:409-432), f32 left-to-right sums."""
    return _mm(lib().ogo_matmul_dequant, ggml_type, raw, in_dim, out_dim, x, n_tokens, threads)


def k_gemm_t(ggml_type, raw, in_dim, out_dim, x, n_tokens) -> np.ndarray:
    """The reference test helper k_gemm (vecdot.rs:4450-4477): yt[out_dim][n_tokens]."""
    raw = _u8(raw)
    x = _f32(x)
    bb, be = BLOCK_LAYOUT[ggml_type]
    row_bytes = in_dim // be * bb
    yt = np.empty((out_dim, n_tokens), np.float32)
    rc = lib().ogo_k_gemm_t(ggml_type, _p(raw), row_bytes, in_dim, out_dim, _p(x), n_tokens, _p(yt))
    if rc != 0:
        raise ValueError(f"ogo_k_gemm_t rc={rc}")
    return yt


def block_sums(ggml_type, raw, in_dim, out_dim, x, n_tokens=1):
    """Integer stage only: isum (and imin for Q4_K and Q5_K) as [n_tokens][out_dim][n_blocks]."""
    raw = _u8(raw)
    x = _f32(x)
    bb, be = BLOCK_LAYOUT[ggml_type]
    row_bytes = in_dim // be * bb
    nb = in_dim // be
    isum = np.zeros((n_tokens, out_dim, nb), np.int32)
    imin = np.zeros((n_tokens, out_dim, nb), np.int32)
    rc = lib().ogo_block_sums(ggml_type, _p(raw), row_bytes, in_dim, out_dim, _p(x), n_tokens,
                              _p(isum), _p(imin))
    if rc != 0:
        raise ValueError(f"ogo_block_sums rc={rc}")
    return isum, imin


def host_threads() -> int:
    return int(lib().ogo_host_threads())

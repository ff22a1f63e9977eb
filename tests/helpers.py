"""Deterministic fixtures shared by the tests.

These restate the reference's own test generators (cited per function) plus the seeded synthetic
generators for the benchmark configurations.  They produce *data*; no arithmetic under test
lives here.
"""
from __future__ import annotations

import numpy as np

Q4_0, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 2, 6, 7, 8, 10, 11, 12, 13, 14, 20, 23
FLAT32 = (Q8_0, Q5_0, Q4_0, IQ4_NL)   # symmetric, one f16 scale per 32 (vecdot.rs:2456-2461)
BLOCK = {Q4_0: (18, 32), Q5_0: (22, 32), Q5_1: (24, 32), Q8_0: (34, 32), Q2_K: (84, 256), Q3_K: (110, 256),
         Q4_K: (144, 256), Q5_K: (176, 256), Q6_K: (210, 256), IQ4_NL: (18, 32), IQ4_XS: (136, 256)}
TYPE_NAME = {Q4_0: "q4_0", Q5_0: "q5_0", Q5_1: "q5_1", Q8_0: "q8_0", Q2_K: "q2_k", Q3_K: "q3_k", Q4_K: "q4_k",
             Q5_K: "q5_k", Q6_K: "q6_k", IQ4_NL: "iq4_nl", IQ4_XS: "iq4_xs"}
# where a block's f16 fields sit: (offset of d, offset of the second field -- dmin or m -- or None)
F16_FIELDS = {Q4_0: (0, None), Q5_0: (0, None), Q5_1: (0, 2), Q8_0: (0, None), IQ4_NL: (0, None), Q2_K: (80, 82),
              Q3_K: (108, None), Q4_K: (0, 2), Q5_K: (0, 2), Q6_K: (208, None), IQ4_XS: (0, None)}


def row_bytes(ggml_type: int, in_dim: int) -> int:
    bb, be = BLOCK[ggml_type]
    assert in_dim % be == 0
    return in_dim // be * bb


def pseudo_bytes(n: int, seed: int) -> np.ndarray:
    """vecdot.rs:3415-3423: s = s*1664525 + 1013904223 (u32), byte = s >> 16."""
    out = np.empty(n, np.uint8)
    s = (seed | 1) & 0xFFFFFFFF
    for i in range(n):
        s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = (s >> 16) & 0xFF
    return out


def pseudo_bytes_fast(n: int, seed: int) -> np.ndarray:
    """Same stream as pseudo_bytes, vectorised (LCG jump-ahead by doubling)."""
    m = 1 << 32
    a, c = 1664525, 1013904223
    # state_k = A_k * s0 + C_k
    A = np.empty(n, np.uint64)
    Cc = np.empty(n, np.uint64)
    A[0], Cc[0] = a, c
    filled = 1
    while filled < n:
        take = min(filled, n - filled)
        # compose: state_{i+filled} = A[filled-1]*state_i + C[filled-1] applied after i steps
        Af, Cf = int(A[filled - 1]), int(Cc[filled - 1])
        A[filled:filled + take] = (A[:take] * np.uint64(Af)) % np.uint64(m)
        Cc[filled:filled + take] = (Cc[:take] * np.uint64(Af) + np.uint64(Cf)) % np.uint64(m)
        filled += take
    s0 = np.uint64((seed | 1) & 0xFFFFFFFF)
    st = (A * s0 + Cc) % np.uint64(m)
    return ((st >> np.uint64(16)) & np.uint64(0xFF)).astype(np.uint8)


def pin_scales(raw: np.ndarray, ggml_type: int) -> np.ndarray:
    """vecdot.rs:3457-3483: overwrite each block's f16 scale fields with finite values
    (d = 0x3000 = 0.125, dmin = 0x2c00 = 0.0625)."""
    bb, _ = BLOCK[ggml_type]
    blocks = raw.reshape(-1, bb)
    if ggml_type in FLAT32:
        blocks[:, 0:2] = (0x00, 0x30)
    elif ggml_type in (Q4_K, Q5_K):   # Q5_K shares Q4_K's leading d / dmin pair (vecdot.rs:3467)
        blocks[:, 0:2] = (0x00, 0x30)
        blocks[:, 2:4] = (0x00, 0x2C)
    elif ggml_type == Q6_K:
        blocks[:, 208:210] = (0x00, 0x30)
    elif ggml_type == Q3_K:   # vecdot.rs:3478
        blocks[:, 108:110] = (0x00, 0x30)
    elif ggml_type == Q5_1:   # vecdot.rs:3462-3465: d then m
        blocks[:, 0:2] = (0x00, 0x30)
        blocks[:, 2:4] = (0x00, 0x2C)
    elif ggml_type == Q2_K:   # vecdot.rs:3472-3475: d then dmin at the end of the block
        blocks[:, 80:82] = (0x00, 0x30)
        blocks[:, 82:84] = (0x00, 0x2C)
    elif ggml_type == IQ4_XS:   # vecdot.rs:3480
        blocks[:, 0:2] = (0x00, 0x30)
    return raw


def fixture_row(ggml_type: int, in_dim: int, seed: int) -> np.ndarray:
    return pin_scales(pseudo_bytes_fast(row_bytes(ggml_type, in_dim), seed), ggml_type)


def k_fixture(ggml_type: int, in_dim: int, out_dim: int, n_tokens: int, seed: int):
    """vecdot.rs:4416-4448: (raw, x)."""
    raw = pin_scales(pseudo_bytes_fast(row_bytes(ggml_type, in_dim) * out_dim, seed), ggml_type)
    i = np.arange(in_dim * n_tokens, dtype=np.int64)
    x = ((i * 37 % 23).astype(np.float32) - np.float32(11.0)) * np.float32(0.031)
    return raw, x.astype(np.float32)


def activations(n: int) -> np.ndarray:
    """vecdot.rs:3425-3429."""
    i = np.arange(n, dtype=np.int64)
    return (((i * 37 % 23).astype(np.float32) - np.float32(11.0)) * np.float32(0.031)).astype(np.float32)


def activations_t(n: int, t: int) -> np.ndarray:
    """vecdot.rs:3716-3721."""
    i = np.arange(n, dtype=np.int64)
    return ((((i * 37 + t * 11) % 23).astype(np.float32) - np.float32(11.0)) * np.float32(0.031)).astype(np.float32)


class NextByte:
    """backend/cpu.rs:515-518: seed = seed*6364136223846793005 + 1 (u64), byte = seed >> 33."""

    def __init__(self, seed: int):
        self.seed = seed & 0xFFFFFFFFFFFFFFFF

    def __call__(self) -> int:
        self.seed = (self.seed * 6364136223846793005 + 1) & 0xFFFFFFFFFFFFFFFF
        return (self.seed >> 33) & 0xFF


def cpu_rs_weights(ggml_type: int, in_dim: int, out_dim: int, nb: NextByte) -> np.ndarray:
    """backend/cpu.rs:587-607 (half::f16::from_f32 rounds to nearest even, as numpy does)."""
    bb, be = BLOCK[ggml_type]
    out = []
    for _ in range(out_dim * (in_dim // be)):
        block = np.zeros(bb, np.uint8)
        scale = np.float32(0.05) + (np.float32(nb()) / np.float32(255.0)) * np.float32(1.95)
        block[0:2] = np.frombuffer(np.float16(scale).tobytes(), np.uint8)
        qf = 2
        if ggml_type in (Q4_K, Q5_K, Q5_1):
            dmin = np.float32(0.05) + (np.float32(nb()) / np.float32(255.0)) * np.float32(0.95)
            block[2:4] = np.frombuffer(np.float16(dmin).tobytes(), np.uint8)
            qf = 4
        for i in range(qf, bb):
            block[i] = nb()
        out.append(block)
    return np.concatenate(out)


# ---------------------------------------------------------------- synthetic benchmark inputs

def synth_weights(ggml_type: int, in_dim: int, out_dim: int, seed: int) -> np.ndarray:
    """Seeded synthetic weights of the benchmark configurations: quant payload uniform random
    bytes, f16 scale fields finite: Q8_0 d = |N(0,0.02)|/127, Q4_K d,dmin = |N(0,0.01)|,
    Q6_K d = |N(0,0.01)|."""
    rng = np.random.default_rng(seed)
    bb, be = BLOCK[ggml_type]
    nblk = out_dim * (in_dim // be)
    raw = rng.integers(0, 256, size=(nblk, bb), dtype=np.uint8)
    if ggml_type == Q8_0:
        q = rng.integers(-127, 128, size=(nblk, 32), dtype=np.int8)
        raw[:, 2:] = q.view(np.uint8)
        d = (np.abs(rng.normal(0, 0.02, nblk)) / 127).astype(np.float16)
        raw[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    elif ggml_type in (Q4_0, Q5_0, IQ4_NL):
        d = (np.abs(rng.normal(0, 0.02, nblk)) / (127 if ggml_type == IQ4_NL else 16)).astype(np.float16)
        raw[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    elif ggml_type == Q5_1:
        d = (np.abs(rng.normal(0, 0.02, nblk)) / 16).astype(np.float16)
        m = rng.normal(0, 0.01, nblk).astype(np.float16)
        raw[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
        raw[:, 2:4] = m.view(np.uint8).reshape(-1, 2)
    elif ggml_type == IQ4_XS:
        d = (np.abs(rng.normal(0, 0.01, nblk)) / 64).astype(np.float16)
        raw[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    elif ggml_type == Q2_K:
        d = np.abs(rng.normal(0, 0.01, nblk)).astype(np.float16)
        dm = np.abs(rng.normal(0, 0.01, nblk)).astype(np.float16)
        raw[:, 80:82] = d.view(np.uint8).reshape(-1, 2)
        raw[:, 82:84] = dm.view(np.uint8).reshape(-1, 2)
    elif ggml_type in (Q4_K, Q5_K):
        d = np.abs(rng.normal(0, 0.01, nblk)).astype(np.float16)
        dm = np.abs(rng.normal(0, 0.01, nblk)).astype(np.float16)
        raw[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
        raw[:, 2:4] = dm.view(np.uint8).reshape(-1, 2)
    else:   # Q6_K, Q3_K: d is the block's last field
        d = np.abs(rng.normal(0, 0.01, nblk)).astype(np.float16)
        raw[:, bb - 2:bb] = d.view(np.uint8).reshape(-1, 2)
    return raw.reshape(-1)


def synth_x(n_tokens: int, in_dim: int, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed ^ 0x5EED)
    return rng.standard_normal((n_tokens, in_dim)).astype(np.float32)

"""CPU restatement of one Llama-family decode step around the quantized matmuls.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's checking
legs, never by the product.

Follows orangu-server's `LlamaModel::run_layers` + `forward` at n_tokens == 1
(engine/arch/llama.rs:594-932, 1007-1032) with the element-wise definitions of engine/tensor.rs
(rmsnorm_into :732-757, rmsnorm_inplace :691-706 per head, add_bias_per_row :1233-1240,
softmax_inplace :809-821, silu :825-827, rope_apply_params_inplace :1115-1177 with NORM or NEOX
pairing and frequency factors; freq_scale 1 and no YaRN, as llama.rs:203-208 sets them), the CPU
attention loop
(engine/attention.rs:426-549), swiglu_ffn_into (engine/arch/mod.rs:1071-1106) and the greedy
argmax (engine/sampling.rs:336-343).  The quantized matmuls are the C oracle's (`oracle.matmul`,
single-token path).

All arithmetic is IEEE f32.  Where the reference adds sequentially (sum of squares, softmax sum,
the weighted sum of V rows) this uses numpy's cumulative sum, which also adds left to right.
`tensor::dot`'s internal accumulator layout is not restated (plain f32 dot): attention scores are
pinned to rounding, not to the bit.

Pinned by tests/test_oracle_llama.py: the reference's own test values (rmsnorm of [3, 4]
tensor.rs:1450-1466, silu(0) / silu(1) :1621-1625, the NORM rotation of [1..8] at position 3
:1752-1769, the NEOX rotation of the same :1731-1749, frequency factors divide the angle
:1785-1822, position 0 = identity :1668, pair norms preserved :1676, softmax sums to one :1612),
closed forms (constant rows, a single cached position, equal scores = mean of V), the grouped-query
head mapping by brute force, and last-of-equal argmax.  parity unpinned: none of these functions
has a bit-level golden vector in the reference; they are pinned to 1e-6.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

f32 = np.float32


def _seq_sum(a: np.ndarray, axis: int = -1) -> np.ndarray:
    """Left-to-right f32 sum (Iterator::sum over f32)."""
    a = np.asarray(a, f32)
    if a.shape[axis] == 0:
        return np.zeros(np.delete(a.shape, axis), f32)
    return np.take(np.cumsum(a, axis=axis, dtype=f32), -1, axis=axis)


def rmsnorm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """tensor.rs:744-749: scale = 1/sqrt(sum(v*v)/dim + eps); out = (v * scale) * w."""
    x = np.asarray(x, f32)
    mean_sq = f32(_seq_sum(x * x) / f32(x.size))
    scale = f32(1.0) / np.sqrt(f32(mean_sq + f32(eps)), dtype=f32)
    return (x * scale).astype(f32) * np.asarray(weight, f32)


_libm = None


def _libm_f32():
    """The C library's single-precision powf, sinf and cosf: what f32::powf and f32::sin_cos
    (tensor.rs:1147, 1160) bind to on Linux.  numpy's float32 power and sin / cos are its own SIMD
    routines and differ from them in the last bit here and there, which at position p turns into
    p ulps of angle; the restatement therefore calls the reference's own functions."""
    global _libm
    if _libm is None:
        import ctypes
        import ctypes.util
        L = ctypes.CDLL(ctypes.util.find_library("m") or "libm.so.6")
        L.powf.restype = ctypes.c_float
        L.powf.argtypes = [ctypes.c_float, ctypes.c_float]
        for fn in (L.sinf, L.cosf):
            fn.restype = ctypes.c_float
            fn.argtypes = [ctypes.c_float]
        _libm = L
    return _libm


def rope_freqs(rope_dim: int, freq_base: float) -> np.ndarray:
    """tensor.rs:1147: freq_i = base.powf(-2 i / rope_dim), in f32."""
    L = _libm_f32()
    expo = (f32(-2.0) * np.arange(rope_dim // 2, dtype=f32) / f32(rope_dim)).astype(f32)
    return np.array([L.powf(float(f32(freq_base)), float(e)) for e in expo], f32)


def rope_sin_cos(theta: np.ndarray):
    """tensor.rs:1160: theta.sin_cos() per pair, in f32."""
    L = _libm_f32()
    t = np.asarray(theta, f32).reshape(-1)
    return (np.array([L.sinf(float(v)) for v in t], f32), np.array([L.cosf(float(v)) for v in t], f32))


def rope(x: np.ndarray, n_head: int, head_dim: int, pos: int, rope_dim: int, freq_base: float,
         freq_factors=None, neox: bool = False) -> np.ndarray:
    """tensor.rs:1115-1177 with freq_scale 1 and ext_factor 0: pair i turns by pos * freq_i, where
    freq_i = base^(-2i / rope_dim) / factor_i (:1147-1150); RopeLayout::Norm pairs elements
    (2i, 2i+1) of every head, RopeLayout::Neox pairs (i, i + rope_dim/2) (:1163-1168)."""
    x = np.array(x, f32).reshape(n_head, head_dim)
    freq = rope_freqs(rope_dim, freq_base)
    if freq_factors is not None:
        freq = (freq / np.asarray(freq_factors, f32)[:rope_dim // 2]).astype(f32)
    theta = (f32(pos) * freq).astype(f32)
    sin, cos = rope_sin_cos(theta)
    half = rope_dim // 2
    lo = slice(0, half) if neox else slice(0, 2 * half, 2)
    hi = slice(half, 2 * half) if neox else slice(1, 2 * half, 2)
    a = x[:, lo].copy()
    b = x[:, hi].copy()
    x[:, lo] = a * cos - b * sin
    x[:, hi] = a * sin + b * cos
    return x.reshape(-1)


def rope_norm(x: np.ndarray, n_head: int, head_dim: int, pos: int, rope_dim: int, freq_base: float) -> np.ndarray:
    """RopeLayout::Norm without frequency factors."""
    return rope(x, n_head, head_dim, pos, rope_dim, freq_base)


def head_rmsnorm(x: np.ndarray, weight: np.ndarray, n_head: int, head_dim: int, eps: float) -> np.ndarray:
    """llama.rs:770-787: rmsnorm_inplace over rows of head_dim, one weight vector for every head."""
    x = np.asarray(x, f32).reshape(n_head, head_dim)
    return np.concatenate([rmsnorm(x[h], weight, eps) for h in range(n_head)])


def softmax(x: np.ndarray) -> np.ndarray:
    """tensor.rs:809-821."""
    x = np.asarray(x, f32)
    e = np.exp((x - x.max()).astype(f32), dtype=f32)
    s = _seq_sum(e)
    return (e / s).astype(f32) if s > 0 else e


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, n_head: int, n_head_kv: int, head_dim: int) -> np.ndarray:
    """attention.rs:426-549 for one token over cache rows k, v [n_pos][n_head_kv*head_dim] (f32
    values): scores = dot(q_h, k_p) / sqrt(head_dim), softmax over positions, out = sum_p w_p v_p
    in ascending position order; query head h reads K/V head h // (n_head / n_head_kv)."""
    q = np.asarray(q, f32).reshape(n_head, head_dim)
    n_pos = k.shape[0]
    k = np.asarray(k, f32).reshape(n_pos, n_head_kv, head_dim)
    v = np.asarray(v, f32).reshape(n_pos, n_head_kv, head_dim)
    group = n_head // n_head_kv
    scale = f32(1.0) / np.sqrt(f32(head_dim), dtype=f32)
    out = np.zeros((n_head, head_dim), f32)
    for h in range(n_head):
        kv = h // group
        scores = ((k[:, kv, :] @ q[h]).astype(f32) * scale).astype(f32)
        w = softmax(scores)
        out[h] = _seq_sum((w[:, None] * v[:, kv, :]).astype(f32), axis=0)
    return out.reshape(-1)


def silu(x: np.ndarray) -> np.ndarray:
    """tensor.rs:825-827: x / (1 + exp(-x))."""
    x = np.asarray(x, f32)
    with np.errstate(over="ignore"):  # exp(-x) = inf for very negative x gives -0, as in the reference
        return (x / (f32(1.0) + np.exp(-x, dtype=f32))).astype(f32)


def to_cache(row: np.ndarray, dtype) -> np.ndarray:
    """A K or V row as the cache keeps it.  The reference's host cache is f32 (kv_cache.rs:75-78); the
    device build keeps f16 and saturates at +-65504 rather than storing an infinity."""
    if dtype == np.float16:
        row = np.clip(row, -65504.0, 65504.0)   # NaN passes through
    return row.astype(dtype)


def argmax(logits: np.ndarray) -> int:
    """sampling.rs:336-343: max_by over f32::total_cmp keeps the last of several equal maxima.
    total_cmp orders -NaN < -inf < ... < -0 < +0 < ... < +inf < +NaN: compare the bit patterns as
    sign-magnitude integers."""
    bits = np.ascontiguousarray(logits, f32).view(np.int32).astype(np.int64)
    keys = np.where(bits < 0, -(bits & 0x7FFFFFFF) - 1, bits)
    return int(np.nonzero(keys == keys.max())[0][-1])


@dataclass
class Layer:
    wq: tuple  # (ggml_type, raw bytes, in_dim, out_dim)
    wk: tuple
    wv: tuple
    wo: tuple
    w_gate: tuple
    w_up: tuple
    w_down: tuple
    attn_norm: np.ndarray
    ffn_norm: np.ndarray
    q_bias: np.ndarray | None = None     # attn_q.bias etc. (Qwen2), llama.rs:174-176
    k_bias: np.ndarray | None = None
    v_bias: np.ndarray | None = None
    q_norm: np.ndarray | None = None     # attn_q_norm.weight etc. (Qwen3), llama.rs:177-178
    k_norm: np.ndarray | None = None


@dataclass
class Model:
    n_embd: int
    n_head: int
    n_head_kv: int
    head_dim: int
    n_ff: int
    n_vocab: int
    rope_dim: int
    rms_eps: float
    rope_freq_base: float
    layers: list
    output_norm: np.ndarray
    output: tuple
    rope_neox: bool = False          # rope_layout_for, llama.rs:115-120
    rope_freq_factors: np.ndarray | None = None   # rope_freqs.weight, llama.rs:186-201
    kv_dtype: type = np.float16      # the build keeps the cache in f16; np.float32 = the reference's host cache
    # kv_hook(layer, pos, k_row, v_row) -> (k_row, v_row): lets a test look at the rows about to be
    # cached and replace them (by a device's rows that differ in the last f16 bit, say)
    kv_hook: object = None
    # act_hook(site, x, group) -> (q, d) or None, at one token only: lets a test look at the f32 input
    # of matmul site `site` (4*layer + 0 q/k/v, + 1 wo, + 2 gate/up, + 3 down; 4*n_layer the output
    # projection) and hand back the quantized activation the matmuls of that site are to use (a
    # device's, which may differ by one unit where an f32 last bit tipped a rounding).  `group` is the
    # quantizer's group of the site's first matrix: 32 or 256.
    act_hook: object = None
    k_cache: list = field(default_factory=list)   # per layer: list of rows
    v_cache: list = field(default_factory=list)

    def reset(self):
        self.k_cache = [[] for _ in self.layers]
        self.v_cache = [[] for _ in self.layers]


def _mm(w: tuple, x: np.ndarray, n_tokens: int = 1) -> np.ndarray:
    """Backend::matmul (cpu.rs:445-458): the GEMV kernels at one token, the GEMM kernels above."""
    import oracle
    t, raw, in_dim, out_dim = w
    y = oracle.matmul(t, raw, in_dim, out_dim, np.ascontiguousarray(x, f32), n_tokens)
    return y.reshape(-1) if n_tokens == 1 else y.reshape(n_tokens, out_dim)


def forward(m: Model, X: np.ndarray, pos0: int, all_rows: bool = False, all_logits: bool = False):
    """llama.rs:594-932 + 1007-1032 for the tokens whose embedding rows are X [n_tokens][n_embd], at
    positions pos0 ..: every matmul over all rows at once, K/V rows appended in order, token t
    attending to cache rows 0 .. pos0 + t; the LAST row alone goes through the output norm and
    projection.  Returns (logits of the last token, its final hidden state); with all_rows instead every
    row after the output norm and no projection (llama.rs:1034-1045); with all_logits the logits of every row
    [n_tokens][n_vocab] and the rows' final hidden states."""
    if not m.k_cache:
        m.reset()
    X = np.array(X, f32).reshape(-1, m.n_embd)
    T = X.shape[0]
    rows = lambda fn, A: np.stack([fn(A[t]) for t in range(T)])

    def mms(site, ws, A):
        """The matmuls of one site over the same input; with an act_hook (one token) they all read the
        quantized activation the hook returns."""
        n_tok = A.shape[0]
        mm = lambda w, A: _mm(w, A if n_tok > 1 else A[0], n_tok).reshape(n_tok, -1)
        if m.act_hook is None or n_tok != 1:
            return [mm(w, A) for w in ws]
        import oracle
        group = 32 if oracle.BLOCK_LAYOUT[ws[0][0]][1] == 32 else 256
        got = m.act_hook(site, A[0], group)
        if got is None:
            return [mm(w, A) for w in ws]
        return [oracle.gemv_act(w[0], w[1], w[2], w[3], got[0], got[1]).reshape(1, -1) for w in ws]

    for li, L in enumerate(m.layers):
        normed = rows(lambda r: rmsnorm(r, L.attn_norm, m.rms_eps), X)
        q, k, v = mms(4 * li, (L.wq, L.wk, L.wv), normed)
        if L.q_bias is not None:                       # llama.rs:757-765
            q = (q + np.asarray(L.q_bias, f32)).astype(f32)
        if L.k_bias is not None:
            k = (k + np.asarray(L.k_bias, f32)).astype(f32)
        if L.v_bias is not None:
            v = (v + np.asarray(L.v_bias, f32)).astype(f32)
        if L.q_norm is not None:                       # llama.rs:770-787, before RoPE
            q = rows(lambda r: head_rmsnorm(r, L.q_norm, m.n_head, m.head_dim, m.rms_eps), q)
        if L.k_norm is not None:
            k = rows(lambda r: head_rmsnorm(r, L.k_norm, m.n_head_kv, m.head_dim, m.rms_eps), k)
        kc, vc = m.k_cache[li], m.v_cache[li]
        assert len(kc) == pos0, "positions must be appended in order"
        attn = np.empty((T, m.n_head * m.head_dim), f32)
        for t in range(T):                             # llama.rs:794-830: one row at a time, in order
            pos = pos0 + t
            qt = rope(q[t], m.n_head, m.head_dim, pos, m.rope_dim, m.rope_freq_base, m.rope_freq_factors, m.rope_neox)
            kt = rope(k[t], m.n_head_kv, m.head_dim, pos, m.rope_dim, m.rope_freq_base, m.rope_freq_factors, m.rope_neox)
            k_row, v_row = to_cache(kt, m.kv_dtype), to_cache(v[t], m.kv_dtype)
            if m.kv_hook is not None:
                k_row, v_row = m.kv_hook(li, pos, k_row, v_row)
            kc.append(k_row)
            vc.append(v_row)
            attn[t] = attention(qt, np.stack(kc).astype(f32), np.stack(vc).astype(f32), m.n_head, m.n_head_kv, m.head_dim)
        X = (X + mms(4 * li + 1, (L.wo,), attn)[0]).astype(f32)
        normed2 = rows(lambda r: rmsnorm(r, L.ffn_norm, m.rms_eps), X)
        gate, up = mms(4 * li + 2, (L.w_gate, L.w_up), normed2)
        h = (silu(gate) * up).astype(f32)
        X = (X + mms(4 * li + 3, (L.w_down,), h)[0]).astype(f32)
    if all_logits:
        # forward_all_logits (arch/mod.rs:2110-2132, composed as gemma.rs:2179-2186): every row through the output
        # norm, one matmul of all rows with the output matrix (the GEMM kernels at more than one row)
        normed = rows(lambda r: rmsnorm(r, m.output_norm, m.rms_eps), X)
        return mms(4 * len(m.layers), (m.output,), normed)[0], X
    if all_rows:
        return rows(lambda r: rmsnorm(r, m.output_norm, m.rms_eps), X)
    last = rmsnorm(X[-1], m.output_norm, m.rms_eps)
    return mms(4 * len(m.layers), (m.output,), last.reshape(1, -1))[0].reshape(-1), X[-1]


def hidden_states(m: Model, X: np.ndarray) -> np.ndarray:
    """forward_hidden_states (llama.rs:1034-1045): run_layers over the tokens from position 0 on a cache
    of its own, then rmsnorm_inplace of every row with the output norm.  [n_tokens][n_embd]."""
    m.reset()
    return forward(m, X, 0, all_rows=True)


def decode_step(m: Model, x: np.ndarray, pos: int):
    """One token: returns (logits, final hidden state)."""
    return forward(m, np.asarray(x, f32).reshape(1, -1), pos)

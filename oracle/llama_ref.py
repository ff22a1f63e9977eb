"""CPU restatement of one Llama-family decode step around the quantized matmuls.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's checking
legs, never by the product.

Follows orangu-server's `LlamaModel::run_layers` + `forward` at n_tokens == 1
(engine/arch/llama.rs:594-932, 1007-1032) with the element-wise definitions of engine/tensor.rs
(rmsnorm_into :732-757, softmax_inplace :809-821, silu :825-827, rope_apply_params_inplace
:1115-1177 with NORM pairing, freq_scale 1, no YaRN, no frequency factors), the CPU attention loop
(engine/attention.rs:426-549), swiglu_ffn_into (engine/arch/mod.rs:1071-1106) and the greedy
argmax (engine/sampling.rs:336-343).  The quantized matmuls are the C oracle's (`oracle.matmul`,
single-token path).

All arithmetic is IEEE f32.  Where the reference adds sequentially (sum of squares, softmax sum,
the weighted sum of V rows) this uses numpy's cumulative sum, which also adds left to right.
`tensor::dot`'s internal accumulator layout is not restated (plain f32 dot): attention scores are
pinned to rounding, not to the bit.

Pinned by tests/test_oracle_llama.py: the reference's own test values (rmsnorm of [3, 4]
tensor.rs:1450-1466, silu(0) / silu(1) :1621-1625, the NORM rotation of [1..8] at position 3
:1752-1769, position 0 = identity :1668, pair norms preserved :1676, softmax sums to one :1612),
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


def rope_freqs(rope_dim: int, freq_base: float) -> np.ndarray:
    """tensor.rs:1147: freq_i = base^(-2i / rope_dim), in f32."""
    i = np.arange(rope_dim // 2, dtype=f32)
    return np.power(f32(freq_base), (f32(-2.0) * i / f32(rope_dim)).astype(f32), dtype=f32)


def rope_norm(x: np.ndarray, n_head: int, head_dim: int, pos: int, rope_dim: int, freq_base: float) -> np.ndarray:
    """tensor.rs:1115-1177, RopeLayout::Norm: pair i is elements (2i, 2i+1) of every head."""
    x = np.array(x, f32).reshape(n_head, head_dim)
    theta = (f32(pos) * rope_freqs(rope_dim, freq_base)).astype(f32)
    sin, cos = np.sin(theta, dtype=f32), np.cos(theta, dtype=f32)
    half = rope_dim // 2
    a = x[:, 0:2 * half:2].copy()
    b = x[:, 1:2 * half:2].copy()
    x[:, 0:2 * half:2] = a * cos - b * sin
    x[:, 1:2 * half:2] = a * sin + b * cos
    return x.reshape(-1)


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


def argmax(logits: np.ndarray) -> int:
    """sampling.rs:336-343: max_by keeps the last of several equal maxima."""
    logits = np.asarray(logits, f32)
    m = logits.max()
    return int(np.nonzero(logits == m)[0][-1])


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
    kv_dtype: type = np.float16      # the build keeps the cache in f16; np.float32 = the reference's host cache
    k_cache: list = field(default_factory=list)   # per layer: list of rows
    v_cache: list = field(default_factory=list)

    def reset(self):
        self.k_cache = [[] for _ in self.layers]
        self.v_cache = [[] for _ in self.layers]


def _mm(w: tuple, x: np.ndarray) -> np.ndarray:
    import oracle
    t, raw, in_dim, out_dim = w
    return oracle.matmul(t, raw, in_dim, out_dim, np.ascontiguousarray(x, f32), 1).reshape(-1)


def decode_step(m: Model, x: np.ndarray, pos: int):
    """llama.rs:594-932 + 1007-1032 for one token.  Returns (logits, final hidden state)."""
    if not m.k_cache:
        m.reset()
    x = np.array(x, f32)
    for li, L in enumerate(m.layers):
        normed = rmsnorm(x, L.attn_norm, m.rms_eps)
        q, k, v = _mm(L.wq, normed), _mm(L.wk, normed), _mm(L.wv, normed)
        q = rope_norm(q, m.n_head, m.head_dim, pos, m.rope_dim, m.rope_freq_base)
        k = rope_norm(k, m.n_head_kv, m.head_dim, pos, m.rope_dim, m.rope_freq_base)
        kc, vc = m.k_cache[li], m.v_cache[li]
        assert len(kc) == pos, "decode positions must be appended in order"
        kc.append(k.astype(m.kv_dtype))
        vc.append(v.astype(m.kv_dtype))
        attn = attention(q, np.stack(kc).astype(f32), np.stack(vc).astype(f32), m.n_head, m.n_head_kv, m.head_dim)
        x = (x + _mm(L.wo, attn)).astype(f32)
        normed2 = rmsnorm(x, L.ffn_norm, m.rms_eps)
        gate, up = _mm(L.w_gate, normed2), _mm(L.w_up, normed2)
        h = (silu(gate) * up).astype(f32)
        x = (x + _mm(L.w_down, h)).astype(f32)
    last = rmsnorm(x, m.output_norm, m.rms_eps)
    return _mm(m.output, last), x

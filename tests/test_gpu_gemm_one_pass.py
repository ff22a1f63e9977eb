"""The one-pass variant of the large-grid K-quant GEMM (tuning key "gemm_one_pass", off by default): Q4_K and
Q5_K fold the reference's separate min pass (vecdot.rs:2229-2240) into the per-super-block step,
`acc += ad * (d * isum - dmin * imin)` -- the single-token expression of vecdot.rs:3152-3178 -- so its f32
results are not the reference GEMM's bits.  What is checked instead:

* against exact arithmetic: the integer sums are rebuilt in numpy int64 from an independent decode of the
  rows, combined in float64, and the kernel must be within a few f32 roundings of that -- a wrong integer
  anywhere is thousands of times the allowance;
* against the reference GEMM's result (the oracle): inside the budget the reference's own tests give its two
  float orders, 1e-3 * sum|w x| (vecdot.rs:3518-3525).  It is NOT everywhere inside 1e-3 relative / 1e-5
  absolute of it, and no other float order can be: both orders sit about 1e-7 of sum|w x| from exact arithmetic
  (printed below; the one-pass order is on average the closer one), each in its own direction, and on an output
  whose terms cancel to near zero that is more than a thousandth of the output.  Hence an option, not the
  default, which keeps the reference's bits.
"""
import sys

import numpy as np
import pytest

import oracle
from helpers import Q4_K, Q5_K, row_bytes, synth_weights, synth_x
from test_oracle_vecdot import np_unpack

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def be():
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()  # raises if the HIP library or the device is missing: no fallback
    b.set_tuning("gemm_min_tokens", 9)
    b.set_tuning("gemm_small_max_tokens", 1)
    b.set_tuning("gemm_plane_cache_mb", 65536)
    b.set_tuning("gemm_plane_kernel", 2)   # the all-waves-multiply kernel whatever the grid
    yield b
    b.close()


def exact_rows(ggml_type, raw, in_dim, rows, x, T):
    """float64 value and magnitude of every (token, sampled row): sum_s ad_s (d_s isum_s - dmin_s imin_s) with
    int64 sums over an independently decoded row, and sum_s |ad_s d_s isum_s| + |ad_s dmin_s imin_s|."""
    nsb = in_dim // 256
    xq = np.empty((T, in_dim), np.int64)
    ad = np.empty((T, nsb), np.float64)
    x = np.asarray(x, np.float32).reshape(T, in_dim)
    for t in range(T):
        q, d, _ = oracle.quantize_act_k_row(x[t])
        xq[t], ad[t] = q, d
    rb = row_bytes(ggml_type, in_dim)
    val = np.empty((T, len(rows)))
    mag = np.empty((T, len(rows)))
    for i, r in enumerate(rows):
        q, sce, mne, d, dmin = np_unpack(ggml_type, raw[r * rb:(r + 1) * rb], in_dim)
        isum = (xq * (q * sce)[None, :]).reshape(T, nsb, 256).sum(axis=2)
        imin = (xq * mne[None, :]).reshape(T, nsb, 256).sum(axis=2)
        pos = ad * d.astype(np.float64)[None, :] * isum
        neg = ad * dmin.astype(np.float64)[None, :] * imin
        val[:, i] = (pos - neg).sum(axis=1)
        mag[:, i] = (np.abs(pos) + np.abs(neg)).sum(axis=1)
    return val, mag


@pytest.mark.parametrize("ggml_type", [Q4_K, Q5_K])
@pytest.mark.parametrize("in_dim,out_dim,T", [(512, 1000, 130), (2048, 300, 257), (256, 129, 33), (4096, 257, 600),
                                              (1024, 64, 2049)])
def test_one_pass_gemm_against_exact_arithmetic_and_the_reference_order(be, ggml_type, in_dim, out_dim, T):
    from orangu_amd import QuantMatrix
    raw = synth_weights(ggml_type, in_dim, out_dim, seed=in_dim + out_dim + T)
    x = synth_x(T, in_dim, seed=T)
    w = QuantMatrix(np.ascontiguousarray(raw), ggml_type, in_dim, out_dim)
    say("one-pass gemm", ggml_type, in_dim, out_dim, T)
    two = np.asarray(be.matmul(x, T, w)).reshape(T, out_dim)
    name = "q4k" if ggml_type == Q4_K else "q5k"
    assert be.last_kernel() == f"ogm_gemm_{name}_dma_kernel"
    be.set_tuning("gemm_one_pass", 1)
    try:
        one = np.asarray(be.matmul(x, T, w)).reshape(T, out_dim)
        assert be.last_kernel() == f"ogm_gemm_{name}_dma_onepass_kernel"
    finally:
        be.set_tuning("gemm_one_pass", 0)
    want = oracle.matmul(ggml_type, raw, in_dim, out_dim, x, T).reshape(T, out_dim)
    assert np.array_equal(two.view(np.uint32), want.view(np.uint32))   # the default stays the reference's bits
    rows = sorted({0, 1, 31, 32, out_dim // 2, out_dim - 33, out_dim - 2, out_dim - 1})
    val, mag = exact_rows(ggml_type, raw, in_dim, rows, x, T)
    nsb = in_dim // 256
    err_one = np.abs(one[:, rows].astype(np.float64) - val)
    err_two = np.abs(two[:, rows].astype(np.float64) - val)
    say("   err / mag: one-pass", (err_one / mag).max(), "two-pass", (err_two / mag).max(),
        "mean abs err: one-pass", err_one.mean(), "two-pass", err_two.mean())
    # three roundings a super-block (d * isum; minus dmin * imin; plus into the accumulator), each half an ulp
    # of something no larger than the magnitude so far
    assert (err_one <= 2.0 ** -24 * (2 + nsb) * mag).all()
    assert err_one.mean() <= err_two.mean()   # closer to exact arithmetic than the reference order
    # the reference's budget between its own two float orders, over every output
    diff = np.abs(one.astype(np.float64) - want.astype(np.float64))
    assert (diff[:, rows] <= 1e-3 * mag).all()
    # and nowhere further from the reference than the rounding noise both carry allows: rows not sampled are
    # bounded through the largest magnitude of the sampled ones (same distribution of weights and inputs)
    assert diff.max() <= 2.0 ** -24 * 4 * (2 + nsb) * mag.max()


def test_one_pass_is_refused_nothing_and_changes_nothing_elsewhere(be):
    """The key only reaches Q4_K / Q5_K on the all-waves-multiply kernel: Q6_K on it, and Q4_K on the
    feeding-wave kernels (a matrix without planes), keep the reference's bits with the key set."""
    from orangu_amd import QuantMatrix
    from helpers import Q6_K
    be.set_tuning("gemm_one_pass", 1)
    try:
        for ggml_type, planes in ((Q6_K, True), (Q4_K, False)):
            in_dim, out_dim, T = 1024, 200, 140
            raw = synth_weights(ggml_type, in_dim, out_dim, seed=5)
            x = synth_x(T, in_dim, seed=6)
            be.set_tuning("gemm_plane_cache_mb", 65536 if planes else 0)
            got = np.asarray(be.matmul(x, T, QuantMatrix(np.ascontiguousarray(raw), ggml_type, in_dim, out_dim)))
            say("   ", be.last_kernel())
            assert "onepass" not in be.last_kernel() and ("_dma_" in be.last_kernel() or "_dmx_" in be.last_kernel()) == planes
            want = oracle.matmul(ggml_type, raw, in_dim, out_dim, x, T)
            assert np.array_equal(got.reshape(-1).view(np.uint32), want.reshape(-1).view(np.uint32))
    finally:
        be.set_tuning("gemm_one_pass", 0)
        be.set_tuning("gemm_plane_cache_mb", 65536)


def test_one_pass_over_several_matrices_in_one_launch(be):
    """gate and up read the same rows and share one launch (arch/mod.rs:1082-1096): with the option on, each
    matrix's result is what the matrix alone gives, bit for bit (the same kernel arithmetic per row tile)."""
    from orangu_amd import MatmulOp, QuantMatrix
    in_dim, T = 1024, 200
    x = synth_x(T, in_dim, seed=3)
    ws = [QuantMatrix(np.ascontiguousarray(synth_weights(Q4_K, in_dim, o, seed=40 + o)), Q4_K, in_dim, o)
          for o in (300, 257, 128)]
    be.set_tuning("gemm_one_pass", 1)
    try:
        alone = []
        for w in ws:
            alone.append(np.asarray(be.matmul(x, T, w)))
            assert be.last_kernel() == "ogm_gemm_q4k_dma_onepass_kernel"
        together = be.matmul_batch([MatmulOp(x, T, w) for w in ws])
        assert be.last_kernel() == "ogm_gemm_q4k_dma_onepass_kernel"
    finally:
        be.set_tuning("gemm_one_pass", 0)
    for a, b in zip(alone, together):
        assert np.array_equal(a.reshape(-1).view(np.uint32), np.asarray(b).reshape(-1).view(np.uint32))


def test_a_prefill_with_one_pass_gemms_holds_the_models_tolerance(be):
    """run_layers over a batch (llama.rs:594-932) with the Q4_K projections' GEMMs in the one-pass order: hidden
    state and logits within the model tests' 2e-4 of the largest magnitude of the CPU restatement, same greedy
    token, and the decode steps after it continue on the cache it wrote."""
    from test_gpu_llama import TAME, build, prefill_both, step_both
    f32 = np.float32
    ref, dev, rng = build(be, n_embd=512, n_head=4, n_kv=2, hd=128, n_ff=1024, n_vocab=320, n_layer=2,
                          types=(Q4_K, Q4_K, Q4_K, Q4_K), max_ctx=256, seed=77, attn_norm_scale=TAME[Q4_K])
    be.set_tuning("gemm_one_pass", 1)
    try:
        X = rng.standard_normal((150, 512)).astype(f32)
        prefill_both(ref, dev, X, 0, "one-pass prefill")
        step_both(ref, dev, rng.standard_normal(512).astype(f32), 150, "then a decode step")
        # the option did reach the batch's GEMMs: the same prompt without it ends in other bits
        one = np.asarray(dev.prefill(X, 0)[0]).copy()
        be.set_tuning("gemm_one_pass", 0)
        two = np.asarray(dev.prefill(X, 0)[0])
        assert not np.array_equal(one.view(np.uint32), two.view(np.uint32))
        assert np.abs(one - two).max() <= 2e-4 * np.abs(two).max()
    finally:
        be.set_tuning("gemm_one_pass", 0)
        dev.close()

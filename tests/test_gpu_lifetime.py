"""What the library allocates, it gives back: contexts, weights (with their prefill planes), decoders with their
KV caches and prefill buffers, created and destroyed over and over, leave the device's free memory where it was
(RocmBackend's Drop frees every cached weight, rocm.rs:609-622)."""
import sys

import numpy as np
import pytest

from helpers import Q4_K, Q6_K, synth_weights, synth_x

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _round(seed):
    from orangu_amd import LlamaDecoder, Mi355xBackend, QuantMatrix
    be = Mi355xBackend()
    try:
        # weights through the cache and without it, single-token and GEMM calls (the latter builds planes)
        ws = [QuantMatrix(np.ascontiguousarray(synth_weights(t, 1024, o, seed=seed + i)), t, 1024, o)
              for i, (t, o) in enumerate(((Q4_K, 2048), (Q6_K, 512), (Q4_K, 4096)))]
        be.set_tuning("gemm_plane_kernel", 2)
        for w in ws:
            be.matmul(synth_x(1, 1024, seed=1), 1, w)
            be.matmul(synth_x(200, 1024, seed=2), 200, w)
        h = be.upload_raw(synth_weights(Q4_K, 1024, 256, seed=3), Q4_K, 1024, 256)
        be.free_weight(h)
        # a decoder: KV cache, a decode step, a prefill (its row buffers), hidden states
        n_embd, n_ff = 256, 512
        mk = lambda t, i, o, s: QuantMatrix(np.ascontiguousarray(synth_weights(t, i, o, seed=s)), t, i, o)
        layers = [{"wq": mk(Q4_K, n_embd, 256, 11), "wk": mk(Q4_K, n_embd, 128, 12), "wv": mk(Q6_K, n_embd, 128, 13),
                   "wo": mk(Q4_K, 256, n_embd, 14), "w_gate": mk(Q4_K, n_embd, n_ff, 15), "w_up": mk(Q4_K, n_embd, n_ff, 16),
                   "w_down": mk(Q6_K, n_ff, n_embd, 17), "attn_norm": np.full(n_embd, 0.02, np.float32),
                   "ffn_norm": np.ones(n_embd, np.float32)} for _ in range(2)]
        dev = LlamaDecoder(be, n_embd=n_embd, n_head=4, n_head_kv=2, head_dim=64, n_ff=n_ff, n_vocab=320, max_ctx=512,
                           rms_eps=1e-5, rope_freq_base=10000.0, layers=layers,
                           output_norm=np.ones(n_embd, np.float32), output=mk(Q6_K, n_embd, 320, 18))
        rng = np.random.default_rng(seed)
        dev.prefill(rng.standard_normal((70, n_embd)).astype(np.float32), 0)
        dev.decode(rng.standard_normal(n_embd).astype(np.float32), 70)
        dev.hidden_states(x=rng.standard_normal((5, n_embd)).astype(np.float32))
        dev.close()
    finally:
        be.close()


def test_repeated_lifetimes_return_the_device_memory():
    from orangu_amd import hiprt
    _round(0)   # the runtime's own pools and code objects are loaded on the first use
    _round(1)
    free0, total = hiprt.mem_get_info()
    for r in range(12):
        _round(2 + r)
    free1, _ = hiprt.mem_get_info()
    say("free before", free0, "after", free1, "of", total)
    # the runtime may keep a few MiB of its own; a leaked weight, plane set or cache would be tens of MiB a round
    assert free0 - free1 < (16 << 20), (free0, free1)

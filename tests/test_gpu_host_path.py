"""Host-pointer calls (Backend::matmul takes host slices, backend/mod.rs:313-366): small ones run their kernels on
pinned staging buffers in place and wait for the results by polling a pinned word that a one-thread kernel behind
them stores, instead of synchronizing the stream.  Every result a caller reads after such a wait must be the
finished one: thousands of calls in a row over changing weights, inputs and shapes, each compared bit for bit
with the CPU path's result for that pair."""
import sys

import numpy as np
import pytest

import oracle
from helpers import Q4_K, Q6_K, Q8_0, synth_weights, synth_x

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def be():
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()  # raises if the HIP library or the device is missing: no fallback
    yield b
    b.close()


def _pairs():
    from orangu_amd import QuantMatrix
    out = []
    for i, (t, in_dim, out_dim, T) in enumerate([(Q4_K, 4096, 1024, 1), (Q6_K, 2048, 300, 1), (Q8_0, 1024, 257, 1),
                                                 (Q4_K, 1024, 4096, 3), (Q6_K, 1024, 64, 8), (Q4_K, 512, 2000, 1),
                                                 (Q4_K, 2048, 640, 12), (Q8_0, 256, 33, 5)]):
        raw = synth_weights(t, in_dim, out_dim, seed=900 + i)
        x = synth_x(T, in_dim, seed=70 + i)
        want = np.asarray(oracle.matmul(t, raw, in_dim, out_dim, x, T), np.float32).reshape(-1)
        out.append((QuantMatrix(np.ascontiguousarray(raw), t, in_dim, out_dim), x, T, want))
    return out


@pytest.mark.parametrize("flag_wait", [1, 0])
def test_a_long_run_of_small_host_calls_reads_finished_results(be, flag_wait):
    pairs = _pairs()
    be.set_tuning("host_flag_wait", flag_wait)
    try:
        rng = np.random.default_rng(4 + flag_wait)
        order = rng.integers(0, len(pairs), 3000)
        say("host calls:", len(order), "flag wait", flag_wait)
        for n, k in enumerate(order):
            w, x, T, want = pairs[k]
            got = np.asarray(be.matmul(x, T, w), np.float32).reshape(-1)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (n, int(k))
    finally:
        be.set_tuning("host_flag_wait", 1)


def test_batches_and_single_calls_interleave(be):
    """matmul_batch (mod.rs:362-366) shares the wait; a batch after single calls and single calls after a batch
    read their own results."""
    from orangu_amd import MatmulOp
    pairs = _pairs()
    for rep in range(300):
        a, b, c = pairs[rep % 8], pairs[(rep + 3) % 8], pairs[(rep + 5) % 8]
        outs = be.matmul_batch([MatmulOp(a[1], a[2], a[0]), MatmulOp(b[1], b[2], b[0])])
        for (w, x, T, want), got in zip((a, b), outs):
            assert np.array_equal(np.asarray(got).reshape(-1).view(np.uint32), want.view(np.uint32)), rep
        got = np.asarray(be.matmul(c[1], c[2], c[0])).reshape(-1)
        assert np.array_equal(got.view(np.uint32), c[3].view(np.uint32)), rep


def test_a_word_that_never_comes_ends_in_a_stream_synchronization(be):
    """The poll is bounded: with the trailing kernel made to store another number (host_flag_wait 2) every call
    runs into the bound, synchronizes the stream after all and still returns the finished result."""
    import time
    pairs = _pairs()
    be.set_tuning("host_flag_wait", 2)
    try:
        for k in (0, 3, 5):
            w, x, T, want = pairs[k]
            t0 = time.perf_counter()
            got = np.asarray(be.matmul(x, T, w), np.float32).reshape(-1)
            dt = time.perf_counter() - t0
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
            assert 0.004 < dt < 1.0, dt
    finally:
        be.set_tuning("host_flag_wait", 1)
    w, x, T, want = pairs[1]
    got = np.asarray(be.matmul(x, T, w), np.float32).reshape(-1)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_several_backends_in_one_process_run_side_by_side():
    """Each context has its own stream, staging buffers and completion word: four of them, each driven by a thread
    of its own over its own weights, return their own results (the reference's backends are per-model objects,
    backend/mod.rs:309-312)."""
    import threading
    from orangu_amd import Mi355xBackend
    pairs = _pairs()
    backends = [Mi355xBackend() for _ in range(4)]
    errors = []

    def worker(k):
        try:
            b = backends[k]
            for n in range(400):
                w, x, T, want = pairs[(n + 2 * k) % len(pairs)]
                got = np.asarray(b.matmul(x, T, w), np.float32).reshape(-1)
                if not np.array_equal(got.view(np.uint32), want.view(np.uint32)):
                    errors.append((k, n))
                    return
        except Exception as e:   # noqa: BLE001 - reported below
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for b in backends:
        b.close()
    assert not errors, errors

"""A seeded walk over (type, in_dim, out_dim, tokens) through a context with no tuning: whatever kernel the
library's own routing picks -- GEMV, chunked GEMV in GEMM order, few-token, small-batch, feeding-wave, flat
or plane kernel -- `matmul` must give every bit of the CPU restatement's matmul (gemm_k_* / dot_flat_pair from
two tokens on, the GEMV forms at one; cpu.rs:445-458) and `matmul_decode` every bit of the GEMV forms per token
(cpu.rs:265-317).  Shapes are drawn around the routing thresholds (token counts 5/6, 16/17, 64/65, 128/129,
256/257; row counts around 64-row tile multiples) and ragged on purpose."""
import numpy as np
import pytest

import oracle
from helpers import BLOCK, TYPE_NAME, pin_scales, pseudo_bytes_fast, row_bytes, synth_weights, synth_x

pytestmark = pytest.mark.gpu

TYPES = sorted(BLOCK)
TOKENS = (1, 2, 3, 5, 6, 8, 9, 16, 17, 31, 32, 33, 63, 64, 65, 100, 128, 129, 200, 256, 257, 300)
ROWS = (1, 2, 31, 33, 63, 64, 65, 127, 129, 200, 257, 500, 700, 1100, 2100, 4100, 8300)


def cases(n, seed, long_rows=False):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        t = TYPES[int(rng.integers(len(TYPES)))]
        elems = BLOCK[t][1]
        if long_rows:   # rows of many blocks: the staging of activations and terms in LDS grows with them
            in_dim = int(rng.choice((8192, 11008, 14336, 16384, 28672))) if elems == 256 else \
                int(rng.choice((8192, 11008, 14336, 16384, 28672, 9248)))
        else:
            in_dim = int(rng.choice((256, 512, 768, 1024, 2048, 2304, 4096, 14336))) if elems == 256 else \
                int(rng.choice((32, 64, 96, 256, 544, 1024, 2048, 4096, 14336)))
        T = int(rng.choice(TOKENS))
        out_dim = int(rng.choice(ROWS))
        if T * out_dim * in_dim > 150e6:     # keeps the CPU side of the whole module within seconds
            out_dim = max(1, int(150e6 // (T * in_dim)))
        out.append(pytest.param(t, in_dim, out_dim, T, i, id=f"{TYPE_NAME[t]}-{in_dim}x{out_dim}-T{T}"))
    return out


@pytest.fixture(scope="module")
def be():
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()  # raises if the HIP library or the device is missing: no fallback
    yield b
    b.close()


def bits(a):
    return np.asarray(a, np.float32).reshape(-1).view(np.uint32)


@pytest.mark.parametrize("t,in_dim,out_dim,T,i", cases(400, 20240611) + cases(150, 977, long_rows=True))
def test_default_routing_is_bit_exact(be, t, in_dim, out_dim, T, i):
    from orangu_amd import QuantMatrix
    if i % 3 == 0:   # arbitrary bytes with finite scales, as the reference's own fixtures are made (vecdot.rs:3436-3526)
        raw = pin_scales(pseudo_bytes_fast(row_bytes(t, in_dim) * out_dim, 1000 + i), t)
    else:
        raw = synth_weights(t, in_dim, out_dim, seed=2000 + i)
    x = synth_x(T, in_dim, seed=3000 + i)
    print("case", TYPE_NAME[t], in_dim, out_dim, T, flush=True)
    w = QuantMatrix(np.ascontiguousarray(raw), t, in_dim, out_dim)
    try:
        got = be.matmul(x, T, w)
        k1 = be.last_kernel()
        want = oracle.matmul(t, raw, in_dim, out_dim, x, T)
        bad = np.nonzero(bits(got) != bits(want))[0]
        assert bad.size == 0, f"matmul via {k1}: {bad.size} of {want.size} differ, first {bad[:4]}"
        got = be.matmul_decode(x, T, w)
        k2 = be.last_kernel()
        want = oracle.matmul_decode(t, raw, in_dim, out_dim, x, T)
        bad = np.nonzero(bits(got) != bits(want))[0]
        assert bad.size == 0, f"matmul_decode via {k2}: {bad.size} of {want.size} differ, first {bad[:4]}"
    finally:
        be.evict(w)


@pytest.mark.parametrize("t,in_dim,out_dim,T,decode", [
    (10, 14336, 33, 32, False),    # Q2_K over per-32 activations: sixteen terms a block, 74 KB of them for one token
    (10, 11008, 70, 5, False),     # ... and 43 blocks a row (tiles one block wide): 176 KB, more than a workgroup can have
    (10, 11008, 130, 40, False),
    (20, 9248, 200, 3, True),      # IQ4_NL, 289 blocks a row: 74 KB of terms for one token in GEMV order
    (8, 9248, 65, 1, False),
])
def test_long_rows_that_outgrow_the_default_lds(be, t, in_dim, out_dim, T, decode):
    """Rows whose staging does not fit the 64 KB a launch aims for: the launch asks for what it needs, and where a
    format of several terms a block meets tiles one block wide, one wave adds a row's terms up in its lanes as the
    column tiles come (the row's own order) instead of keeping them all.  Same bits as ever."""
    from orangu_amd import QuantMatrix
    raw = synth_weights(t, in_dim, out_dim, seed=in_dim + out_dim)
    x = synth_x(T, in_dim, seed=T)
    w = QuantMatrix(np.ascontiguousarray(raw), t, in_dim, out_dim)
    be.set_tuning("gemm_min_tokens", 100000)   # (batches of these sizes would take a matrix-core kernel)
    try:
        if decode:
            got, want = be.matmul_decode(x, T, w), oracle.matmul_decode(t, raw, in_dim, out_dim, x, T)
        else:
            got, want = be.matmul(x, T, w), oracle.matmul(t, raw, in_dim, out_dim, x, T)
        assert be.last_kernel().startswith("ogm_gemv_kernel"), be.last_kernel()
        bad = np.nonzero(bits(got) != bits(want))[0]
        assert bad.size == 0, f"{be.last_kernel()}: {bad.size} of {want.size} differ, first {bad[:4]}"
    finally:
        be.set_tuning("gemm_min_tokens", 0)
        be.evict(w)


def _batches(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        n_ops = int(rng.integers(1, 7))
        in_dims = [int(rng.choice((256, 512, 1024, 2048, 4096))) for _ in range(2)]
        ops = []
        for _ in range(n_ops):
            t = TYPES[int(rng.integers(len(TYPES)))]
            ops.append((t, in_dims[int(rng.integers(2))], int(rng.choice((1, 31, 64, 65, 129, 300, 1100))),
                        int(rng.integers(3))))          # which of three inputs of that width it reads
        T = int(rng.choice((0, 1, 2, 5, 6, 8, 9, 17, 40, 70, 130)))
        out.append(pytest.param(ops, T, bool(rng.integers(2)), int(rng.choice((0, 0, 16, 64))), i, id=f"batch{i}-{n_ops}ops-T{T}"))
    return out


@pytest.mark.parametrize("ops,T,decode,stripe,i", _batches(60, 31337))
def test_batches_of_mixed_ops_are_bit_exact(be, ops, T, decode, stripe, i):
    """matmul_batch / matmul_batch_decode (mod.rs:362-366, 405) over ops of mixed types and widths, several of
    which share an input (they are quantized once and grouped into one launch where their type allows), with
    token stripes (mod.rs:154-172) and empty ops in between: every op's result is that of its own matmul."""
    from orangu_amd import MatmulOp, QuantMatrix
    xs = {}
    ms, want = [], []
    for k, (t, in_dim, out_dim, which) in enumerate(ops):
        n_tok = 0 if (k == 1 and i % 5 == 0) else T      # now and then an op of no tokens in front of others
        key = (in_dim, which, n_tok)
        if key not in xs:
            xs[key] = synth_x(max(n_tok, 1), in_dim, seed=5000 + 10 * i + which)[:n_tok]
        raw = synth_weights(t, in_dim, out_dim, seed=6000 + 10 * i + k)
        w = QuantMatrix(np.ascontiguousarray(raw), t, in_dim, out_dim)
        ms.append(MatmulOp(xs[key], n_tok, w))
        if n_tok == 0:
            want.append(np.zeros(0, np.float32))
        else:
            # a striped op is the backend's matmul of every stripe (guarded_matmul_op, mod.rs:154-172): a last
            # stripe of one token takes the single-token forms
            step = stripe if (stripe and not decode) else n_tok
            fn = oracle.matmul_decode if decode else oracle.matmul
            want.append(np.concatenate([
                np.asarray(fn(t, raw, in_dim, out_dim, np.ascontiguousarray(xs[key][s0:s0 + step]), min(step, n_tok - s0))).reshape(-1)
                for s0 in range(0, n_tok, step)]))
    print("batch", i, [(TYPE_NAME[o[0]], o[1], o[2], o[3]) for o in ops], "T", T, "decode", decode, "stripe", stripe, flush=True)
    try:
        got = be.matmul_batch_decode(ms) if decode else be.matmul_batch(ms, stripe)
        for k, (g, w_) in enumerate(zip(got, want)):
            bad = np.nonzero(bits(g) != bits(w_))[0] if w_.size else np.zeros(0)
            assert np.asarray(g).size == w_.size and bad.size == 0, f"op {k} {ops[k]}: {bad.size} of {w_.size} differ (last kernel {be.last_kernel()})"
    finally:
        for m in ms:
            be.evict(m.w)


def _large_grids(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        t = int(rng.choice((10, 11, 12, 13, 14, 23, 8)))
        in_dim = int(rng.choice((256, 512, 1024)))
        out_dim = int(rng.choice((16600, 20000, 33000, 41000)))
        T = int(rng.choice((3, 4, 9, 16, 130, 260, 390)))
        if T * out_dim * in_dim > 3e9:
            T = max(3, int(3e9 // (out_dim * in_dim)))
        out.append(pytest.param(t, in_dim, out_dim, T, i, id=f"{TYPE_NAME[t]}-{in_dim}x{out_dim}-T{T}"))
    return out


@pytest.mark.parametrize("t,in_dim,out_dim,T,i", _large_grids(16, 555))
def test_default_routing_on_matrices_of_many_rows(be, t, in_dim, out_dim, T, i):
    """Row counts at which the launches outnumber the compute units: the few-token kernel's default range (Q6_K from
    30 000 rows, 3 to 16 tokens) and the grids of more than 256 tiles of 128 x 128 that go to the plane kernel whose
    waves all multiply, next to the kernels the other types take there."""
    from orangu_amd import QuantMatrix
    raw = synth_weights(t, in_dim, out_dim, seed=7000 + i)
    x = synth_x(T, in_dim, seed=8000 + i)
    w = QuantMatrix(np.ascontiguousarray(raw), t, in_dim, out_dim)
    print("case", TYPE_NAME[t], in_dim, out_dim, T, flush=True)
    try:
        got = be.matmul(x, T, w)
        k1 = be.last_kernel()
        want = oracle.matmul(t, raw, in_dim, out_dim, x, T)
        bad = np.nonzero(bits(got) != bits(want))[0]
        assert bad.size == 0, f"matmul via {k1}: {bad.size} of {want.size} differ, first {bad[:4]}"
        print("  via", k1, flush=True)
        if T <= 16:
            got = be.matmul_decode(x, T, w)
            want = oracle.matmul_decode(t, raw, in_dim, out_dim, x, T)
            bad = np.nonzero(bits(got) != bits(want))[0]
            assert bad.size == 0, f"matmul_decode via {be.last_kernel()}: {bad.size} of {want.size} differ"
    finally:
        be.evict(w)


def _medium_grids(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        t = int(rng.choice((11, 12, 13, 14)))
        in_dim = int(rng.choice((256, 512, 1024, 2048)))
        out_dim = int(rng.choice((2100, 3100, 4100, 6200, 8300))) + int(rng.integers(-70, 70))
        T = int(rng.choice((97, 129, 161, 192, 224, 257, 300, 385, 513, 641)))
        if T * out_dim * in_dim > 3e9:
            in_dim = 256 * max(1, int(3e9 // (T * out_dim * 256)))
        out.append(pytest.param(t, in_dim, out_dim, T, i, id=f"{TYPE_NAME[t]}-{in_dim}x{out_dim}-T{T}"))
    return out


MEDIUM_GRID_KERNELS = set()


@pytest.mark.parametrize("t,in_dim,out_dim,T,i", _medium_grids(40, 4242))
def test_default_routing_on_medium_grids(be, t, in_dim, out_dim, T, i):
    """One to five token tiles of 128 over 33 to 130 row tiles of 64: where, by the size of the launch, the K-quants
    leave the small-batch kernel for the medium-batch kernel, the plane kernel with 64-row tiles, the feeding-wave
    kernels or the plane kernel with 128-row tiles.  Every bit of the CPU GEMM's (vecdot.rs:2213-2303, 2352-2398),
    whichever runs."""
    from orangu_amd import QuantMatrix
    raw = synth_weights(t, in_dim, out_dim, seed=9000 + i)
    x = synth_x(T, in_dim, seed=9500 + i)
    w = QuantMatrix(np.ascontiguousarray(raw), t, in_dim, out_dim)
    print("case", TYPE_NAME[t], in_dim, out_dim, T, flush=True)
    try:
        got = be.matmul(x, T, w)
        k1 = be.last_kernel()
        MEDIUM_GRID_KERNELS.add(k1)
        want = oracle.matmul(t, raw, in_dim, out_dim, x, T)
        bad = np.nonzero(bits(got) != bits(want))[0]
        assert bad.size == 0, f"matmul via {k1}: {bad.size} of {want.size} differ, first {bad[:4]}"
        print("  via", k1, flush=True)
    finally:
        be.evict(w)


def test_medium_grids_reached_every_kernel_family():
    """The walk above is only worth its time if it lands on the kernels it is there for."""
    if not MEDIUM_GRID_KERNELS:
        pytest.skip("the walk did not run in this process")
    names = " ".join(sorted(MEDIUM_GRID_KERNELS))
    for piece in ("_dmx_kernel", "_dma_kernel", "ogm_gemm_sbw_", "_r64_kernel", "ogm_gemm_sb_"):
        assert piece in names, (piece, names)

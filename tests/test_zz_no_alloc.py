"""The entry point that allocates nothing (ogm_matmul_dev_static) against ogm_matmul_dev, through
the C ABI: same bits, on calls in a row that share the GPU's static scratch array, the later ones
smaller than the first; sizes beyond the array are refused; and nothing is allocated (free device memory and
the context's scratch unchanged across the calls, from a fresh context on)."""
import numpy as np
import pytest

from helpers import Q4_K, Q6_K, Q8_0, synth_weights, synth_x

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    from orangu_amd import Mi355xBackend
    b = Mi355xBackend()
    yield b
    b.close()


def both(be, hiprt, stream, handle, x, T, out_dim, decode):
    """(ogm_matmul_dev_static, ogm_matmul_dev) outputs for the same device-resident input."""
    xd = hiprt.DeviceBuffer.from_numpy(x)
    y1, y2 = hiprt.DeviceBuffer(4 * T * out_dim), hiprt.DeviceBuffer(4 * T * out_dim)
    y1.fill(0xFF)
    y2.fill(0xFF)
    be.matmul_dev_static(handle, xd.ptr, T, y1.ptr, decode, stream.ptr)
    be.matmul_dev(handle, xd.ptr, T, y2.ptr, decode, stream.ptr)
    stream.synchronize()
    got, want = y1.to_numpy(np.float32, T * out_dim), y2.to_numpy(np.float32, T * out_dim)
    for b in (xd, y1, y2):
        b.free()
    return got, want


def test_static_scratch_entry_equals_matmul_dev_on_calls_in_a_row(be):
    import oracle
    from orangu_amd import hiprt
    stream = hiprt.Stream()
    # the first call is the largest; the ones after it are smaller and find its leftovers in the array
    calls = [(Q4_K, 14336, 96, 8, False), (Q4_K, 4096, 130, 3, False), (Q4_K, 4096, 130, 1, False),
             (Q6_K, 4096, 70, 4, True), (Q8_0, 4096, 65, 8, False), (Q8_0, 1024, 33, 1, True),
             (Q6_K, 14336, 40, 1, False), (Q4_K, 256, 3, 2, False)]
    for n, (t, in_dim, out_dim, T, decode) in enumerate(calls):
        raw = synth_weights(t, in_dim, out_dim, seed=90 + n)
        x = synth_x(T, in_dim, seed=190 + n)
        h = be.upload_raw(raw, t, in_dim, out_dim)
        try:
            got, want = both(be, hiprt, stream, h, x, T, out_dim, decode)
        finally:
            be.free_weight(h)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (n, t, in_dim, out_dim, T, decode)
        cpu = (oracle.matmul_decode if decode else oracle.matmul)(t, raw, in_dim, out_dim, x, T).reshape(-1)
        assert np.all(np.abs(got.astype(np.float64) - cpu) <= 1e-3 * np.abs(cpu) + 1e-5), (n, "against the CPU path")
    stream.destroy()


def test_static_scratch_entry_allocates_nothing(be):
    """The defining property: on a fresh context, whose grown-on-demand scratch is still empty, calls in a row --
    the largest the array admits first -- leave the device's free memory and the context's scratch where they were."""
    from orangu_amd import Mi355xBackend, hiprt
    fresh = Mi355xBackend()
    stream = hiprt.Stream()
    shapes = [(Q4_K, 32768, 40, 8, False), (Q6_K, 14336, 70, 8, True), (Q8_0, 4096, 65, 3, False),
              (Q4_K, 4096, 130, 1, False)]
    held = []
    try:
        for n, (t, in_dim, out_dim, T, decode) in enumerate(shapes):
            h = fresh.upload_raw(synth_weights(t, in_dim, out_dim, seed=300 + n), t, in_dim, out_dim)
            xd = hiprt.DeviceBuffer.from_numpy(synth_x(T, in_dim, seed=400 + n))
            yd = hiprt.DeviceBuffer(4 * T * out_dim)
            held.append((h, xd, yd, T, decode))
        # warm-up on another context: the runtime loads a kernel's code on its first launch in a process
        for h, xd, yd, T, decode in held:
            be.matmul_dev_static(h, xd.ptr, T, yd.ptr, decode, stream.ptr)
        stream.synchronize()
        hiprt.device_synchronize()
        assert fresh.scratch_bytes() == 0          # nothing has run on this context yet
        free0 = hiprt.mem_get_info()[0]
        for _ in range(2):
            for h, xd, yd, T, decode in held:
                fresh.matmul_dev_static(h, xd.ptr, T, yd.ptr, decode, stream.ptr)
        stream.synchronize()
        assert fresh.scratch_bytes() == 0
        assert hiprt.mem_get_info()[0] == free0
        # the allocating entry point on the same inputs does grow the scratch: the check above can see a regression
        h, xd, yd, T, decode = held[0]
        fresh.matmul_dev(h, xd.ptr, T, yd.ptr, decode, stream.ptr)
        stream.synchronize()
        assert fresh.scratch_bytes() > 0
    finally:
        for h, xd, yd, _, _ in held:
            fresh.free_weight(h)
            xd.free()
            yd.free()
        stream.destroy()
        fresh.close()


def test_static_scratch_entry_refuses_what_does_not_fit(be):
    from orangu_amd import OgmError, hiprt
    raw = synth_weights(Q4_K, 4096, 16, seed=5)
    h = be.upload_raw(raw, Q4_K, 4096, 16)
    wide = be.upload_raw(synth_weights(Q4_K, 36864, 2, seed=6), Q4_K, 36864, 2)
    xd, yd = hiprt.DeviceBuffer(4 * 9 * 36864), hiprt.DeviceBuffer(4 * 9 * 16)
    xd.fill(0)
    yd.fill(0x7F)
    try:
        with pytest.raises(OgmError, match="static scratch"):
            be.matmul_dev_static(h, xd.ptr, 9, yd.ptr)            # more than 8 tokens
        with pytest.raises(OgmError, match="static scratch"):
            be.matmul_dev_static(wide, xd.ptr, 8, yd.ptr)         # 8 * 36864 activations > 262144
        be.matmul_dev_static(wide, xd.ptr, 7, yd.ptr)             # 7 * 36864 fit
        hiprt.device_synchronize()
        be.matmul_dev_static(h, xd.ptr, 0, yd.ptr)                # nothing to do
    finally:
        be.free_weight(h)
        be.free_weight(wide)
        xd.free()
        yd.free()

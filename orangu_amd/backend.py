"""Host-side mirror of the reference's backend seam, over the C ABI.

Same names and argument meaning as ``engine::backend::Backend``
(src/bin/orangu-server/engine/backend/mod.rs:309-496), ``MatmulOp`` (mod.rs:121-125) and
``QuantMatrix`` (engine/loader.rs:561-680), so the parity tests read like the reference's own
(engine/backend/cpu.rs:509-651, engine/backend/rocm.rs:633-697).  Every method runs the HIP
kernels through ``liborangu_mi355x.so``; there is no CPU path here.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import capi
from .capi import OgmError, OgmOp

BLOCK_LAYOUT = {2: (18, 32), 6: (22, 32), 7: (24, 32), 8: (34, 32), 10: (84, 256), 11: (110, 256), 12: (144, 256),
                13: (176, 256), 14: (210, 256), 20: (18, 32), 23: (136, 256)}

# backend/mod.rs:304-306
MATMUL_ONLY_SURFACE = "matmul only - no fused layer chain, GPU attention or GPU sampling"
# backend/mod.rs:131
MAX_MULTI_TOKEN_PHASE_TOKENS_DEFAULT = 256


class QuantMatrix:
    """A quantized weight matrix as the loader hands it to a backend: ``out_dim`` contiguous rows
    of ``row_bytes`` raw GGUF blocks (engine/loader.rs:561-680)."""

    def __init__(self, data, ggml_type: int, in_dim: int, out_dim: int, start: int = 0):
        self._bytes = np.ascontiguousarray(
            np.frombuffer(data, dtype=np.uint8) if isinstance(data, (bytes, bytearray)) else data,
            dtype=np.uint8)
        if ggml_type not in BLOCK_LAYOUT:
            raise ValueError(f"unsupported ggml_type {ggml_type}")
        bb, be = BLOCK_LAYOUT[ggml_type]
        if in_dim % be != 0:
            raise ValueError(f"in_dim {in_dim} is not a multiple of the block size {be}")
        self._ggml_type = ggml_type
        self._start = start
        self._row_bytes = in_dim // be * bb
        self.in_dim = in_dim
        self.out_dim = out_dim
        if start + self._row_bytes * out_dim > self._bytes.size:
            raise ValueError("byte range exceeds the tensor")  # loader.rs:1562-1570

    def ggml_type(self) -> int:
        return self._ggml_type

    def row_bytes(self) -> int:
        return self._row_bytes

    def raw_bytes(self) -> np.ndarray:
        return self._bytes[self._start:self._start + self._row_bytes * self.out_dim]

    def rows(self, first: int, count: int) -> "QuantMatrix":
        """loader.rs:627-646: a view of rows first..first+count sharing the same bytes."""
        if first + count > self.out_dim:
            raise ValueError(f"row range {first}..{first + count} exceeds out_dim {self.out_dim}")
        return QuantMatrix(self._bytes, self._ggml_type, self.in_dim, count,
                           self._start + first * self._row_bytes)

    def cache_key(self) -> tuple[int, int]:
        """loader.rs:674-679: (absolute address, byte length)."""
        return (self._bytes.ctypes.data + self._start, self._row_bytes * self.out_dim)


@dataclass
class MatmulOp:
    """backend/mod.rs:121-125."""
    x: np.ndarray
    n_tokens: int
    w: QuantMatrix


class Mi355xBackend:
    """``impl Backend`` over the MI355X kernels."""

    def __init__(self, device: int = 0):
        self._lib = capi.load_library()
        ctx = C.c_void_p()
        rc = self._lib.ogm_init(device, C.byref(ctx))
        if rc != 0:
            raise OgmError(rc, "ogm_init", self._lib.ogm_last_error(None).decode())
        self._ctx = ctx
        self._keepalive: dict[tuple[int, int], np.ndarray] = {}

    # ---- lifetime ----
    @classmethod
    def try_init(cls, device: int = 0):
        """RocmBackend::try_init (rocm.rs:168-173): None when no usable device."""
        try:
            return cls(device)
        except OgmError:
            return None

    def close(self):
        if getattr(self, "_ctx", None):
            self._lib.ogm_destroy(self._ctx)
            self._ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc: int, where: str):
        if rc != 0:
            raise OgmError(rc, where, self._lib.ogm_last_error(self._ctx).decode())

    def device_name(self) -> str:
        buf = C.create_string_buffer(256)
        self._check(self._lib.ogm_device_name(self._ctx, buf, 256), "ogm_device_name")
        return buf.value.decode()

    # ---- Backend ----
    def supports_type(self, ggml_type: int) -> bool:
        return bool(self._lib.ogm_supports_type(ggml_type))

    def reduced_surface(self):
        return MATMUL_ONLY_SURFACE

    def as_wgpu(self):
        return None

    def upload(self, w: QuantMatrix) -> int:
        """Weight handle for ``w``, uploading (and repacking) on first sight of its cache key."""
        key = w.cache_key()
        raw = w.raw_bytes()
        handle = C.c_void_p()
        rc = self._lib.ogm_weight_upload(self._ctx, w.ggml_type(), raw.ctypes.data, w.row_bytes(),
                                         w.in_dim, w.out_dim, key[0], key[1], C.byref(handle))
        self._check(rc, "ogm_weight_upload")
        self._keepalive[key] = w._bytes  # the key is an address: keep the bytes alive with it
        return handle.value

    def download(self, w: QuantMatrix) -> np.ndarray:
        h = self.upload(w)
        out = np.empty(w.row_bytes() * w.out_dim, np.uint8)
        self._check(self._lib.ogm_weight_download(self._ctx, h, out.ctypes.data, out.size),
                    "ogm_weight_download")
        return out

    def _x(self, x, n_tokens: int, w: QuantMatrix) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
        if x.size != n_tokens * w.in_dim:
            raise ValueError(f"x has {x.size} elements, expected {n_tokens}*{w.in_dim}")
        return x

    def matmul(self, x, n_tokens: int, w: QuantMatrix) -> np.ndarray:
        """y[t, o] = sum_i x[t, i] * w.row(o)[i]; returns [n_tokens * out_dim] (mod.rs:313)."""
        out = np.empty(0, np.float32)
        return self.matmul_into(out, x, n_tokens, w)

    def matmul_into(self, out: np.ndarray, x, n_tokens: int, w: QuantMatrix) -> np.ndarray:
        x = self._x(x, n_tokens, w)
        y = np.empty(n_tokens * w.out_dim, np.float32)
        h = self.upload(w)
        self._check(self._lib.ogm_matmul(self._ctx, h, x.ctypes.data, n_tokens, y.ctypes.data), "ogm_matmul")
        return y

    def matmul_decode(self, x, n_tokens: int, w: QuantMatrix) -> np.ndarray:
        """mod.rs:386: the single-token kernel per (row, token)."""
        x = self._x(x, n_tokens, w)
        y = np.empty(n_tokens * w.out_dim, np.float32)
        h = self.upload(w)
        self._check(self._lib.ogm_matmul_decode(self._ctx, h, x.ctypes.data, n_tokens, y.ctypes.data),
                    "ogm_matmul_decode")
        return y

    def _batch(self, ops, decode: bool, max_tokens: int):
        arr = (OgmOp * len(ops))()
        xs, ys = [], []
        for i, op in enumerate(ops):
            x = self._x(op.x, op.n_tokens, op.w)
            y = np.empty(op.n_tokens * op.w.out_dim, np.float32)
            xs.append(x)
            ys.append(y)
            arr[i].w = self.upload(op.w)
            arr[i].x = x.ctypes.data
            arr[i].n_tokens = op.n_tokens
            arr[i].y = y.ctypes.data
        self._check(self._lib.ogm_matmul_batch(self._ctx, arr, len(ops), int(decode), max_tokens),
                    "ogm_matmul_batch")
        return ys

    def matmul_batch(self, ops, max_tokens_per_phase: int = 0):
        """mod.rs:362-366: independent ops; long ones run in token stripes (mod.rs:154-172)."""
        return self._batch(ops, False, max_tokens_per_phase)

    def matmul_batch_decode(self, ops):
        """mod.rs:405."""
        return self._batch(ops, True, 0)

    # ---- integer stage, for parity checks ----
    def quantize_act(self, x, per_256: bool):
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        n = x.size
        g = 256 if per_256 else 32
        q = np.empty(n, np.int8)
        d = np.empty(n // g, np.float32)
        s = np.empty(n // 16, np.int32)
        self._check(self._lib.ogm_quantize_act(self._ctx, int(per_256), x.ctypes.data, n,
                                               q.ctypes.data, d.ctypes.data, s.ctypes.data),
                    "ogm_quantize_act")
        return q, d, s

    def quantize_act_tokens(self, x, in_dim: int, n_tokens: int, per_256: bool):
        """The quantizer over a batch as the multi-token matmuls launch it: token-major
        (q [T][in], d [T][in/group], sums [T][in/16], bsum [T][in/32], bs16 [T][in/16] or None)."""
        x = np.ascontiguousarray(x, np.float32).reshape(n_tokens, in_dim)
        g = 256 if per_256 else 32
        q = np.empty((n_tokens, in_dim), np.int8)
        d = np.empty((n_tokens, in_dim // g), np.float32)
        s = np.empty((n_tokens, in_dim // 16), np.int32)
        b = np.empty((n_tokens, in_dim // 32), np.int16)
        h = np.empty((n_tokens, in_dim // 16), np.uint16) if per_256 else None
        self._check(self._lib.ogm_quantize_act_tokens(self._ctx, int(per_256), x.ctypes.data, in_dim, n_tokens,
                                                      q.ctypes.data, d.ctypes.data, s.ctypes.data, b.ctypes.data,
                                                      h.ctypes.data if h is not None else None),
                    "ogm_quantize_act_tokens")
        return q, d, s, b, h

    def dump_block_sums(self, x, n_tokens: int, w: QuantMatrix):
        x = self._x(x, n_tokens, w)
        _, be = BLOCK_LAYOUT[w.ggml_type()]
        shape = (n_tokens, w.out_dim, w.in_dim // be)
        isum = np.zeros(shape, np.int32)
        imin = np.zeros(shape, np.int32)
        h = self.upload(w)
        self._check(self._lib.ogm_dump_block_sums(self._ctx, h, x.ctypes.data, n_tokens,
                                                  isum.ctypes.data, imin.ctypes.data),
                    "ogm_dump_block_sums")
        return isum, imin

    def f16_to_f32(self, bits) -> np.ndarray:
        bits = np.ascontiguousarray(bits, np.uint16)
        out = np.empty(bits.size, np.float32)
        self._check(self._lib.ogm_f16_to_f32(self._ctx, bits.ctypes.data, bits.size, out.ctypes.data),
                    "ogm_f16_to_f32")
        return out

    # ---- device-resident path (torch tensors or raw device pointers) ----
    def matmul_dev(self, w_handle: int, x_ptr: int, n_tokens: int, y_ptr: int, decode: bool = False,
                   stream: int = 0):
        self._check(self._lib.ogm_matmul_dev(self._ctx, w_handle, x_ptr, n_tokens, y_ptr,
                                             int(decode), stream or None), "ogm_matmul_dev")

    def matmul_dev_static(self, w_handle: int, x_ptr: int, n_tokens: int, y_ptr: int, decode: bool = False,
                          stream: int = 0):
        """ogm_matmul_dev without any allocation: the library's static device scratch takes the
        quantized activations (at most 8 tokens and 262144 activations per call)."""
        self._check(self._lib.ogm_matmul_dev_static(self._ctx, w_handle, x_ptr, n_tokens, y_ptr,
                                                    int(decode), stream or None), "ogm_matmul_dev_static")

    def act_quantize_dev(self, ggml_type: int, x_ptr: int, in_dim: int, n_tokens: int, stream: int = 0,
                         decode: bool = False):
        """Quantizes device-resident x for following matmul_act_dev calls: with decode=False in matmul's activation
        mode, with decode=True in matmul_decode's (they differ for Q2_K at several tokens only)."""
        fn = self._lib.ogm_act_quantize_decode_dev if decode else self._lib.ogm_act_quantize_dev
        self._check(fn(self._ctx, ggml_type, x_ptr, in_dim, n_tokens, stream or None),
                    "ogm_act_quantize_decode_dev" if decode else "ogm_act_quantize_dev")

    def matmul_act_dev(self, w_handle: int, n_tokens: int, y_ptr: int, decode: bool = False,
                       stream: int = 0):
        self._check(self._lib.ogm_matmul_act_dev(self._ctx, w_handle, n_tokens, y_ptr, int(decode),
                                                 stream or None), "ogm_matmul_act_dev")

    def matmul_multi_dev(self, w_handles, x_ptr: int, n_tokens: int, y_ptrs, decode: bool = False,
                         stream: int = 0):
        """Several weights over one device-resident input (q/k/v, gate/up): one quantize, and at
        one token one launch."""
        n = len(w_handles)
        ws = (C.c_void_p * n)(*w_handles)
        ys = (C.c_void_p * n)(*y_ptrs)
        self._check(self._lib.ogm_matmul_multi_dev(self._ctx, ws, n, x_ptr, n_tokens, ys, int(decode),
                                                   stream or None), "ogm_matmul_multi_dev")

    def matmul_multi_act_dev(self, w_handles, n_tokens: int, y_ptrs, decode: bool = False, stream: int = 0):
        """The grouped call over activations quantized by act_quantize_dev."""
        n = len(w_handles)
        ws = (C.c_void_p * n)(*w_handles)
        ys = (C.c_void_p * n)(*y_ptrs)
        self._check(self._lib.ogm_matmul_multi_act_dev(self._ctx, ws, n, n_tokens, ys, int(decode),
                                                       stream or None), "ogm_matmul_multi_act_dev")

    def time_host_calls(self, variants, group_sizes, reps: int) -> np.ndarray:
        """Wall time in microseconds of `reps` repetitions of host-pointer calls issued from compiled
        code: `variants` is a list of equally long lists of MatmulOp (repetition r takes variants[r %
        len]), walked in groups of `group_sizes` ops -- one op: ogm_matmul, several: ogm_matmul_batch."""
        n_ops = len(variants[0])
        arr = (OgmOp * (n_ops * len(variants)))()
        keep = []
        for v, ops in enumerate(variants):
            assert len(ops) == n_ops
            for i, op in enumerate(ops):
                x = self._x(op.x, op.n_tokens, op.w)
                y = np.empty(op.n_tokens * op.w.out_dim, np.float32)
                keep += [x, y]
                a = arr[v * n_ops + i]
                a.w, a.x, a.n_tokens, a.y = self.upload(op.w), x.ctypes.data, op.n_tokens, y.ctypes.data
        gs = (C.c_uint32 * len(group_sizes))(*group_sizes)
        out = (C.c_double * reps)()
        self._check(self._lib.ogm_time_host_calls(self._ctx, arr, n_ops, len(variants), gs, len(group_sizes), reps, out),
                    "ogm_time_host_calls")
        return np.array(out[:], np.float64)

    def weights_read_probe(self, w_handles, stream: int = 0):
        """One launch that only reads the device bytes of 1..4 uploaded weights (for benchmarks)."""
        n = len(w_handles)
        ws = (C.c_void_p * n)(*w_handles)
        self._check(self._lib.ogm_weights_read_probe(self._ctx, ws, n, stream or None), "ogm_weights_read_probe")

    def empty_launch(self, workgroups: int, stream: int = 0):
        """One launch of `workgroups` workgroups that does nothing (for benchmarks: a kernel boundary)."""
        self._check(self._lib.ogm_empty_launch(self._ctx, workgroups, stream or None), "ogm_empty_launch")

    def enqueue_repeated(self, kind: int, w_sets, n_tokens: int, y_ptrs, first: int, reps: int, decode: bool = False,
                         stream: int = 0):
        """`reps` launches back to back from compiled code, rotating over `w_sets` (equally long lists of weight
        handles) from set `first`: kind 0 the grouped GEMV over quantized activations, 1 the read-only probe,
        2 empty launches of n_tokens workgroups (w_sets and y_ptrs unused)."""
        n_var = max(1, len(w_sets))
        n_ws = len(w_sets[0]) if w_sets else 0
        flat = [h for s in w_sets for h in s]
        ws = (C.c_void_p * max(1, len(flat)))(*flat)
        ys = (C.c_void_p * max(1, len(y_ptrs)))(*y_ptrs)
        self._check(self._lib.ogm_enqueue_repeated(self._ctx, kind, ws, n_ws, n_var, n_tokens, ys, int(decode),
                                                   first, reps, stream or None), "ogm_enqueue_repeated")

    def scratch_bytes(self) -> int:
        """Bytes of device and pinned scratch the context has grown so far (weights not counted)."""
        return int(self._lib.ogm_scratch_bytes(self._ctx))

    def upload_raw(self, raw: np.ndarray, ggml_type: int, in_dim: int, out_dim: int) -> int:
        """Uploads without a cache key: every call makes a new device copy."""
        raw = np.ascontiguousarray(raw, np.uint8)
        bb, be = BLOCK_LAYOUT[ggml_type]
        handle = C.c_void_p()
        rc = self._lib.ogm_weight_upload(self._ctx, ggml_type, raw.ctypes.data, in_dim // be * bb,
                                         in_dim, out_dim, 0, 0, C.byref(handle))
        self._check(rc, "ogm_weight_upload")
        return handle.value

    def free_weight(self, w_handle: int):
        """Releases a device copy made by upload_raw (cached uploads live as long as the backend)."""
        self._check(self._lib.ogm_weight_free(self._ctx, w_handle), "ogm_weight_free")

    def evict(self, w: QuantMatrix):
        """Frees the device copy of ``w`` and forgets its cache key.  The reference's backends never
        evict (engine/backend/rocm.rs:329-350); tests that build multi-gigabyte models do."""
        self.free_weight(self.upload(w))
        self._keepalive.pop(w.cache_key(), None)

    def dequant_rows(self, w, row0: int, n_rows: int, in_dim: int | None = None) -> np.ndarray:
        """Rows of an uploaded matrix (a QuantMatrix, or a handle together with its in_dim) as f32,
        from the device copy (quant.rs dequantize_*)."""
        handle = w if isinstance(w, int) else self.upload(w)
        out = np.empty((n_rows, in_dim if isinstance(w, int) else w.in_dim), np.float32)
        self._check(self._lib.ogm_dequant_rows(self._ctx, handle, row0, n_rows, out.ctypes.data),
                    "ogm_dequant_rows")
        return out

    def set_tuning(self, key: str, value: int):
        self._check(self._lib.ogm_set_tuning(self._ctx, key.encode(), value), "ogm_set_tuning")

    def last_kernel(self) -> str:
        return self._lib.ogm_last_kernel(self._ctx).decode()

    def argmax(self, logits: np.ndarray) -> int:
        """sampling::argmax (engine/sampling.rs:336-343) on the device: the decode step's greedy pick."""
        logits = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
        out = C.c_uint32(0)
        self._check(self._lib.ogm_argmax(self._ctx, logits.ctypes.data, logits.size, C.byref(out)), "ogm_argmax")
        return int(out.value)


class LlamaDecoder:
    """The device-resident decode step of a Llama-family model over a Mi355xBackend
    (LlamaModel::forward at n_tokens == 1, engine/arch/llama.rs:1007-1032).

    ``layers`` is a list of dicts with QuantMatrix entries wq, wk, wv, wo, w_gate, w_up, w_down,
    f32 arrays attn_norm, ffn_norm and, where the file has them, q_bias, k_bias, v_bias (Qwen2) and
    q_norm, k_norm (Qwen3; llama.rs:174-178); ``output`` a QuantMatrix; ``output_norm`` an f32 array.
    ``rope_neox`` follows rope_layout_for (llama.rs:115-120): False for "llama" / "mistral" files;
    ``rope_freq_factors`` is rope_freqs.weight (llama.rs:186-201) or None."""

    def __init__(self, be: "Mi355xBackend", *, n_embd: int, n_head: int, n_head_kv: int, head_dim: int,
                 n_ff: int, n_vocab: int, layers, output_norm, output, max_ctx: int, rope_dim: int | None = None,
                 rms_eps: float = 1e-5, rope_freq_base: float = 10000.0, rope_neox: bool = False,
                 rope_freq_factors=None, upload=None):
        self._be = be
        up = upload or be.upload
        rope_dim = head_dim if rope_dim is None else rope_dim
        self._keep = []
        ff = None
        if rope_freq_factors is not None:
            ff = np.ascontiguousarray(rope_freq_factors, np.float32).reshape(-1)
            if ff.size < rope_dim // 2:   # llama.rs:189-195
                raise ValueError(f"rope_freq_factors has {ff.size} entries, need {rope_dim // 2}")
            self._keep.append(ff)
        cfg = capi.OgmLlamaConfig(len(layers), n_embd, n_head, n_head_kv, head_dim, n_ff, n_vocab,
                                  rope_dim, max_ctx, rms_eps, rope_freq_base, 1 if rope_neox else 0,
                                  ff.ctypes.data if ff is not None else None)
        arr = (capi.OgmLlamaLayer * len(layers))()
        want = {"q_bias": n_head * head_dim, "k_bias": n_head_kv * head_dim, "v_bias": n_head_kv * head_dim,
                "q_norm": head_dim, "k_norm": head_dim}
        for i, L in enumerate(layers):
            for name in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down"):
                setattr(arr[i], name, up(L[name]))
            for name in ("attn_norm", "ffn_norm"):
                a = np.ascontiguousarray(L[name], np.float32)
                self._keep.append(a)
                setattr(arr[i], name, a.ctypes.data)
            for name, size in want.items():
                if L.get(name) is None:
                    continue
                a = np.ascontiguousarray(L[name], np.float32).reshape(-1)
                if a.size != size:
                    raise ValueError(f"layer {i}: {name} has {a.size} values, expected {size}")
                self._keep.append(a)
                setattr(arr[i], name, a.ctypes.data)
        on = np.ascontiguousarray(output_norm, np.float32)
        h = C.c_void_p()
        be._check(be._lib.ogm_llama_create(be._ctx, C.byref(cfg), arr, on.ctypes.data, up(output), C.byref(h)),
                  "ogm_llama_create")
        self._h = h.value
        self.n_embd, self.n_vocab, self.kv_dim, self.n_layer = n_embd, n_vocab, n_head_kv * head_dim, len(layers)
        self._act_width = max(n_embd, n_ff, n_head * head_dim)

    @classmethod
    def from_gguf(cls, be: "Mi355xBackend", gguf, max_ctx: int) -> "LlamaDecoder":
        """The decoder of a Llama-style GGUF file (a ``GgufFile``), built by the library as
        LlamaModel::load_with_backend builds the model (llama.rs:123-220).  ``tok_embd`` is the
        uploaded embedding matrix's handle, for ``generate`` and ``Mi355xBackend.dequant_rows``."""
        self = cls.__new__(cls)
        self._be, self._keep = be, [gguf]
        h, embd, cfg = C.c_void_p(), C.c_void_p(), capi.OgmLlamaConfig()
        rc = be._lib.ogm_llama_load_gguf(be._ctx, gguf._h, max_ctx, C.byref(h), C.byref(embd), C.byref(cfg))
        if rc != 0:
            gguf._fail(rc, "ogm_llama_load_gguf")
        self._h, self.tok_embd, self.config = h.value, embd.value, cfg
        self.n_embd, self.n_vocab, self.n_layer = cfg.n_embd, cfg.n_vocab, cfg.n_layer
        self.kv_dim = cfg.n_head_kv * cfg.head_dim
        self._act_width = max(cfg.n_embd, cfg.n_ff, cfg.n_head * cfg.head_dim)
        return self

    def kv_write(self, layer: int, pos0: int, k, v):
        k = np.ascontiguousarray(k, np.float32).reshape(-1, self.kv_dim)
        v = np.ascontiguousarray(v, np.float32).reshape(-1, self.kv_dim)
        self._be._check(self._be._lib.ogm_llama_kv_write(self._be._ctx, self._h, layer, pos0, k.shape[0],
                                                         k.ctypes.data, v.ctypes.data), "ogm_llama_kv_write")

    def kv_read(self, layer: int, pos0: int, n_pos: int):
        """Cache rows pos0 .. pos0+n_pos of a layer as float16 arrays [n_pos][kv_dim] (k, v)."""
        k = np.empty((n_pos, self.kv_dim), np.float16)
        v = np.empty((n_pos, self.kv_dim), np.float16)
        self._be._check(self._be._lib.ogm_llama_kv_read(self._be._ctx, self._h, layer, pos0, n_pos,
                                                        k.ctypes.data, v.ctypes.data), "ogm_llama_kv_read")
        return k, v

    def decode(self, x, pos: int):
        """Returns (logits, argmax) for the token whose embedding row is x, at position pos."""
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        if x.size != self.n_embd:
            raise ValueError(f"x has {x.size} values, n_embd = {self.n_embd}")
        logits = np.empty(self.n_vocab, np.float32)
        am = C.c_uint32()
        self._be._check(self._be._lib.ogm_llama_decode(self._be._ctx, self._h, x.ctypes.data, pos,
                                                       logits.ctypes.data, C.byref(am)), "ogm_llama_decode")
        return logits, am.value

    def prefill(self, x, pos0: int = 0):
        """Returns (logits, argmax) of the last of the tokens whose embedding rows are x
        [n_tokens][n_embd], placed at positions pos0 .. (run_layers at n_tokens > 1)."""
        x = np.ascontiguousarray(x, np.float32).reshape(-1, self.n_embd)
        logits = np.empty(self.n_vocab, np.float32)
        am = C.c_uint32()
        self._be._check(self._be._lib.ogm_llama_prefill(self._be._ctx, self._h, x.ctypes.data, pos0, x.shape[0],
                                                        logits.ctypes.data, C.byref(am)), "ogm_llama_prefill")
        return logits, am.value

    def forward_all_logits(self, x=None, pos0: int = 0, tok_embd=None, tokens=None, want_logits: bool = True):
        """Model::forward_all_logits (arch/mod.rs:2110-2132): the positions' embedding rows x [n][n_embd] (or token
        ids into tok_embd) appended at pos0; returns (logits [n][n_vocab] or None, greedy token of every position)."""
        if (x is None) == (tok_embd is None):
            raise ValueError("give embedding rows or a matrix with token ids")
        if x is not None:
            x = np.ascontiguousarray(x, np.float32).reshape(-1, self.n_embd)
            n, xp, hp, tp = x.shape[0], x.ctypes.data, None, None
        else:
            hp = tok_embd if isinstance(tok_embd, int) else self._be.upload(tok_embd)
            tokens = np.ascontiguousarray(tokens, np.uint32).reshape(-1)
            n, xp, tp = tokens.size, None, tokens.ctypes.data
        logits = np.empty((n, self.n_vocab), np.float32) if want_logits else None
        am = np.empty(n, np.uint32)
        self._be._check(self._be._lib.ogm_llama_forward_all_logits(
            self._be._ctx, self._h, xp, hp, tp, pos0, n, logits.ctypes.data if want_logits else None, am.ctypes.data),
            "ogm_llama_forward_all_logits")
        return logits, am

    def prefill_tokens(self, tok_embd, tokens, pos0: int = 0):
        """The same from token ids; tok_embd is a QuantMatrix [n_embd -> n_vocab] or a handle."""
        h = tok_embd if isinstance(tok_embd, int) else self._be.upload(tok_embd)
        tokens = np.ascontiguousarray(tokens, np.uint32).reshape(-1)
        logits = np.empty(self.n_vocab, np.float32)
        am = C.c_uint32()
        self._be._check(self._be._lib.ogm_llama_prefill_tokens(self._be._ctx, self._h, h, tokens.ctypes.data, pos0,
                                                               tokens.size, logits.ctypes.data, C.byref(am)),
                        "ogm_llama_prefill_tokens")
        return logits, am.value

    def hidden_states(self, x=None, tok_embd=None, tokens=None) -> np.ndarray:
        """forward_hidden_states (llama.rs:1034-1045): [n_tokens][n_embd], every token's final hidden state
        after the output norm, from embedding rows x or from token ids into tok_embd (a QuantMatrix or a
        handle).  Starts from position 0 and overwrites the model's cache rows."""
        if (x is None) == (tok_embd is None):
            raise ValueError("give embedding rows or a matrix with token ids")
        if x is not None:
            x = np.ascontiguousarray(x, np.float32).reshape(-1, self.n_embd)
            n, xp, hp, tp = x.shape[0], x.ctypes.data, None, None
        else:
            hp = tok_embd if isinstance(tok_embd, int) else self._be.upload(tok_embd)
            tokens = np.ascontiguousarray(tokens, np.uint32).reshape(-1)
            n, xp, tp = tokens.size, None, tokens.ctypes.data
        out = np.empty((n, self.n_embd), np.float32)
        self._be._check(self._be._lib.ogm_llama_hidden_states(self._be._ctx, self._h, xp, hp, tp, n, out.ctypes.data),
                        "ogm_llama_hidden_states")
        return out

    def decode_dev(self, x_ptr: int, pos: int, logits_ptr: int = 0, argmax_ptr: int = 0, stream: int = 0):
        self._be._check(self._be._lib.ogm_llama_decode_dev(self._be._ctx, self._h, x_ptr, pos, logits_ptr or None,
                                                           argmax_ptr or None, stream or None), "ogm_llama_decode_dev")

    def generate(self, tok_embd, first_token: int, pos0: int, n_tokens: int, want_logits: bool = False):
        """Greedy generation on the device; tok_embd is a QuantMatrix [n_embd -> n_vocab] or a handle."""
        h = tok_embd if isinstance(tok_embd, int) else self._be.upload(tok_embd)
        toks = np.empty(n_tokens, np.uint32)
        logits = np.empty(self.n_vocab, np.float32) if want_logits else None
        self._be._check(self._be._lib.ogm_llama_generate(self._be._ctx, self._h, h, first_token, pos0, n_tokens,
                                                         toks.ctypes.data, logits.ctypes.data if want_logits else None),
                        "ogm_llama_generate")
        return (toks, logits) if want_logits else toks

    def hidden(self) -> np.ndarray:
        out = np.empty(self.n_embd, np.float32)
        self._be._check(self._be._lib.ogm_llama_debug_hidden(self._be._ctx, self._h, out.ctypes.data),
                        "ogm_llama_debug_hidden")
        return out

    def attn_stamps(self, n_workgroups: int) -> np.ndarray:
        """Timeline builds only: [n_workgroups][8] wall-clock stamps (100 MHz) of the last attention launch."""
        out = np.zeros((n_workgroups, 8), np.uint64)
        self._be._check(self._be._lib.ogm_debug_attn_stamps(self._be._ctx, out.ctypes.data, out.size),
                        "ogm_debug_attn_stamps")
        return out

    def capture_acts(self, on: bool = True):
        """Debug: keep the quantized activations every matmul group of a decode step reads."""
        self._be._check(self._be._lib.ogm_llama_debug_capture(self._be._ctx, self._h, 1 if on else 0),
                        "ogm_llama_debug_capture")

    def act(self, site: int):
        """(q int8 [n], d f32 [n / group], group) of matmul site ``site`` of the last decode step:
        4*layer + 0 q/k/v input, + 1 wo input, + 2 gate/up input, + 3 down input; 4*n_layer the output
        projection's input."""
        q = np.empty(self._act_width, np.int8)
        d = np.empty(self._act_width // 32 + 1, np.float32)
        n, group = C.c_uint32(0), C.c_uint32(0)
        self._be._check(self._be._lib.ogm_llama_debug_act(self._be._ctx, self._h, site, q.ctypes.data, d.ctypes.data,
                                                          C.byref(n), C.byref(group)), "ogm_llama_debug_act")
        return q[:n.value].copy(), d[:n.value // group.value].copy(), int(group.value)

    def close(self):
        if self._h:
            self._be._lib.ogm_llama_destroy(self._be._ctx, self._h)
            self._h = None

"""frink_amd -- MI355X (gfx950) quantized-matmul backend for Frink: Python binding of the C ABI.

The product is ``lib/libfrink_hip.so`` (HIP kernels + C ABI, ``include/frink_hip.h``).  This
module only loads it with ctypes and passes device pointers of torch tensors through; torch is
used for device memory and streams, nothing else.  There is no CPU fallback: if the library is
missing or no gfx950 device answers, calls raise.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfrink_hip.so")

# quant kinds (ggml type ids) and their QuantKind::name()
Q4_0, Q8_0, Q4_K, Q5_K, Q6_K = 2, 8, 12, 13, 14
Q5_0, IQ4_XS, MXFP4 = 6, 23, 39
KIND_NAME = {Q4_0: "Q4_0", Q8_0: "Q8_0", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", Q5_0: "Q5_0", IQ4_XS: "IQ4_XS", MXFP4: "MXFP4"}
BLOCK = {Q4_0: (18, 32), Q8_0: (34, 32), Q4_K: (144, 256), Q5_K: (176, 256), Q6_K: (210, 256),
         Q5_0: (22, 32), IQ4_XS: (136, 256), MXFP4: (17, 32)}  # (block_bytes, block_elems)
ACT_F32, ACT_INT8, ACT_F32_DOT = 0, 1, 2

OK, ERR_NO_DEVICE, ERR_UNSUPPORTED, ERR_SHAPE, ERR_ARG, ERR_HIP, ERR_OOM = 0, -1, -2, -3, -4, -5, -6

EXPORTS = [
    "frk_hip_probe", "frk_hip_dense_enabled", "frk_hip_last_error", "frk_hip_matvec_kernel",
    "frk_hip_gemm_supported", "frk_hip_has_launch", "frk_hip_block_bytes", "frk_hip_block_elems",
    "frk_hip_worth_a_gemm", "frk_hip_weights_register", "frk_hip_weights_from_device",
    "frk_hip_weights_release", "frk_hip_weights_keep_decoded", "frk_hip_weights_rows", "frk_hip_weights_cols", "frk_hip_weights_kind",
    "frk_hip_launch_matvec", "frk_hip_launch_mul_mm", "frk_hip_launch_matvec_multi",
    "frk_hip_launch_dense_ffn_swiglu", "frk_hip_gemv_multi_dev", "frk_hip_ffn_swiglu_dev", "frk_hip_gemv_dev", "frk_hip_gemv_q8k_dev",
    "frk_hip_gemm_dev", "frk_hip_gemm_q8k_dev", "frk_hip_gemm_pair_dev", "frk_hip_gemm_noalloc_dev",
    "frk_hip_batch_acts_create", "frk_hip_batch_acts_release", "frk_hip_quantize_batch_acts_dev", "frk_hip_gemm_acts_dev", "frk_hip_route_top_k_softmax_dev", "frk_hip_moe_ffn_dev",
    "frk_hip_moe_intermediates_dev",
    "frk_hip_quantize_q8_k_dev", "frk_hip_quantize_q8_0_dev", "frk_hip_dequant_dev",
    "frk_hip_get_rows_dev", "frk_hip_get_rows",
    "frk_hip_copy_dev", "frk_hip_read_dev", "frk_hip_issue_probe", "frk_hip_read_shape_dev", "frk_hip_gemm_grouped_dev",
]


class BackendError(RuntimeError):
    """A failed call; carries the C ABI's status code and message
    (the reference's BackendError, crates/frink-core/src/weight_matrix/gpu_backend.rs:90)."""

    def __init__(self, code, message):
        super().__init__("%s (status %d)" % (message, code))
        self.code = code
        self.message = message


class DeviceInfo(C.Structure):
    _fields_ = [("device_count", C.c_int32), ("compute_units", C.c_int32), ("name", C.c_char * 128),
                ("gcn_arch", C.c_char * 64), ("total_vram_bytes", C.c_uint64), ("free_vram_bytes", C.c_uint64)]


_lib = None


def lib():
    """The loaded C ABI library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python -m frink_amd.build`" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        vp, sz, i = C.c_void_p, C.c_size_t, C.c_int
        sig = {
            "frk_hip_probe": (i, [C.POINTER(DeviceInfo)]),
            "frk_hip_dense_enabled": (i, []),
            "frk_hip_last_error": (C.c_char_p, []),
            "frk_hip_matvec_kernel": (C.c_char_p, [i]),
            "frk_hip_gemm_supported": (i, [i]),
            "frk_hip_has_launch": (i, [i]),
            "frk_hip_block_bytes": (i, [i]),
            "frk_hip_block_elems": (i, [i]),
            "frk_hip_worth_a_gemm": (i, [sz]),
            "frk_hip_weights_register": (i, [i, vp, sz, sz, sz, C.POINTER(vp)]),
            "frk_hip_weights_from_device": (i, [i, vp, sz, sz, sz, vp, C.POINTER(vp)]),
            "frk_hip_weights_release": (i, [vp]),
            "frk_hip_weights_keep_decoded": (i, [vp, vp]),
            "frk_hip_weights_rows": (sz, [vp]),
            "frk_hip_weights_cols": (sz, [vp]),
            "frk_hip_weights_kind": (i, [vp]),
            "frk_hip_launch_matvec": (i, [i, vp, sz, vp, sz, sz, sz, vp]),
            "frk_hip_launch_mul_mm": (i, [i, vp, sz, vp, sz, sz, sz, sz, sz, vp]),
            "frk_hip_launch_matvec_multi": (i, [vp, sz, vp, sz, vp]),
            "frk_hip_launch_dense_ffn_swiglu": (i, [vp, vp, vp, vp, sz, vp]),
            "frk_hip_gemv_multi_dev": (i, [vp, sz, vp, vp, vp]),
            "frk_hip_ffn_swiglu_dev": (i, [vp, vp, vp, vp, vp, vp]),
            "frk_hip_gemv_dev": (i, [vp, vp, vp, i, vp]),
            "frk_hip_gemv_q8k_dev": (i, [vp, vp, vp, vp, vp, vp]),
            "frk_hip_gemm_dev": (i, [vp, vp, sz, vp, vp]),
            "frk_hip_gemm_q8k_dev": (i, [vp, vp, vp, vp, sz, vp, vp]),
            "frk_hip_gemm_noalloc_dev": (i, [vp, vp, sz, vp, vp]),
            "frk_hip_gemm_pair_dev": (i, [vp, vp, vp, sz, vp, vp, vp]),
            "frk_hip_batch_acts_create": (i, [sz, sz, C.POINTER(vp)]),
            "frk_hip_batch_acts_release": (i, [vp]),
            "frk_hip_quantize_batch_acts_dev": (i, [vp, vp, sz, vp]),
            "frk_hip_gemm_acts_dev": (i, [vp, vp, vp, vp]),
            "frk_hip_route_top_k_softmax_dev": (i, [vp, sz, sz, sz, i, vp, vp, vp]),
            "frk_hip_moe_ffn_dev": (i, [vp, vp, vp, sz, vp, sz, vp, vp, sz, vp, vp]),
            "frk_hip_moe_intermediates_dev": (i, [sz, sz, sz, sz, sz, vp, vp, vp, vp, vp, vp]),
            "frk_hip_quantize_q8_k_dev": (i, [vp, sz, vp, vp, vp, vp]),
            "frk_hip_quantize_q8_0_dev": (i, [vp, sz, vp, vp, vp]),
            "frk_hip_dequant_dev": (i, [vp, vp, vp]),
            "frk_hip_get_rows_dev": (i, [vp, vp, C.c_size_t, vp, vp]),
            "frk_hip_get_rows": (i, [vp, vp, C.c_size_t, vp]),
            "frk_hip_copy_dev": (i, [vp, vp, sz, vp]),
            "frk_hip_read_dev": (i, [vp, sz, vp, vp]),
            "frk_hip_issue_probe": (i, [vp]),
            "frk_hip_gemm_grouped_dev": (i, [vp, sz, vp, vp, vp, sz, sz, vp, vp]),
            "frk_hip_read_shape_dev": (i, [vp, sz, vp, i, i, i, i, vp]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error():
    return lib().frk_hip_last_error().decode()


def check(status):
    if status != OK:
        raise BackendError(status, last_error())


def probe():
    """Device facts, or raises BackendError(ERR_NO_DEVICE) on a host without a gfx950 GPU."""
    info = DeviceInfo()
    check(lib().frk_hip_probe(C.byref(info)))
    return {"device_count": info.device_count, "compute_units": info.compute_units,
            "name": info.name.decode(), "gcn_arch": info.gcn_arch.decode(),
            "total_vram_bytes": info.total_vram_bytes, "free_vram_bytes": info.free_vram_bytes}


def matvec_kernel(kind):
    r = lib().frk_hip_matvec_kernel(kind)
    return r.decode() if r else None


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _np_ptr(a):
    return C.c_void_p(a.ctypes.data)


class Weights:
    """One quantized weight matrix resident in HBM (the reference's
    WeightMatrix::Quantized{data, rows, cols, kind}, crates/frink-core/src/weight_matrix.rs:780-787)."""

    def __init__(self, handle, kind, rows, cols, keepalive=None):
        self.handle, self.kind, self.rows, self.cols = handle, kind, rows, cols
        self._keepalive = keepalive

    @classmethod
    def from_host(cls, kind, data, rows, cols):
        data = np.ascontiguousarray(np.frombuffer(data, np.uint8) if isinstance(data, (bytes, bytearray)) else data,
                                    dtype=np.uint8)
        h = C.c_void_p()
        check(lib().frk_hip_weights_register(kind, _np_ptr(data), data.size, rows, cols, C.byref(h)))
        return cls(h, kind, rows, cols, keepalive=data)

    @classmethod
    def from_device(cls, kind, data_dev, rows, cols):
        """data_dev: a uint8 torch tensor on the GPU holding GGUF block bytes."""
        h = C.c_void_p()
        check(lib().frk_hip_weights_from_device(kind, C.c_void_p(data_dev.data_ptr()), data_dev.numel(), rows, cols,
                                                _stream(), C.byref(h)))
        return cls(h, kind, rows, cols)

    def keep_decoded(self):
        """Q5_0 / IQ4_XS / MXFP4: keep the rows decoded for the matrix cores beside the resident copy."""
        check(lib().frk_hip_weights_keep_decoded(self.handle, _stream()))
        return self

    def release(self):
        if self.handle:
            check(lib().frk_hip_weights_release(self.handle))
            self.handle = None

    def __del__(self):
        try:
            if self.handle and _lib is not None:
                _lib.frk_hip_weights_release(self.handle)
                self.handle = None
        except Exception:
            pass

    # ---- device-resident operations (torch tensors on cuda:0) ----
    def gemv(self, x, out=None, act_mode=ACT_F32):
        import torch
        assert x.dtype == torch.float32 and x.is_cuda and x.is_contiguous() and x.numel() == self.cols
        y = out if out is not None else torch.empty(self.rows, dtype=torch.float32, device=x.device)
        check(lib().frk_hip_gemv_dev(self.handle, C.c_void_p(x.data_ptr()), C.c_void_p(y.data_ptr()), act_mode,
                                     _stream()))
        return y

    def gemv_q8k(self, acts, out=None):
        """acts = (q, d, bsums) from quantize_q8_k: one activation shared by several projections."""
        import torch
        q, d, bs = acts
        y = out if out is not None else torch.empty(self.rows, dtype=torch.float32, device=q.device)
        check(lib().frk_hip_gemv_q8k_dev(self.handle, C.c_void_p(q.data_ptr()), C.c_void_p(d.data_ptr()),
                                         C.c_void_p(bs.data_ptr()), C.c_void_p(y.data_ptr()), _stream()))
        return y

    def gemm_q8k(self, acts, batch, out=None):
        """A thin batch over activations quantized beforehand: acts = (q, d, bsums) of quantize_q8_k over the batch."""
        import torch
        q, d, bs = acts
        y = out if out is not None else torch.empty((batch, self.rows), dtype=torch.float32, device=q.device)
        check(lib().frk_hip_gemm_q8k_dev(self.handle, C.c_void_p(q.data_ptr()), C.c_void_p(d.data_ptr()),
                                         C.c_void_p(bs.data_ptr()), batch, C.c_void_p(y.data_ptr()), _stream()))
        return y

    def gemm(self, x, out=None):
        import torch
        assert x.dtype == torch.float32 and x.is_cuda and x.is_contiguous() and x.shape[-1] == self.cols
        batch = x.numel() // self.cols
        y = out if out is not None else torch.empty((batch, self.rows), dtype=torch.float32, device=x.device)
        check(lib().frk_hip_gemm_dev(self.handle, C.c_void_p(x.data_ptr()), batch, C.c_void_p(y.data_ptr()),
                                     _stream()))
        return y

    def gemm_acts(self, acts, out=None):
        """apply_batch_with_acts: this matrix over a batch that a BatchActs holds quantized."""
        import torch
        y = out if out is not None else torch.empty((acts.batch, self.rows), dtype=torch.float32, device="cuda")
        check(lib().frk_hip_gemm_acts_dev(self.handle, acts.handle, C.c_void_p(y.data_ptr()), _stream()))
        return y

    def gemm_noalloc(self, x, out):
        """frk_hip_gemm_noalloc_dev: the caller brings the output; the call allocates nothing."""
        import torch
        assert x.dtype == torch.float32 and x.is_cuda and x.is_contiguous() and x.shape[-1] == self.cols
        batch = x.numel() // self.cols
        assert out.dtype == torch.float32 and out.is_cuda and out.is_contiguous() and out.numel() == batch * self.rows
        check(lib().frk_hip_gemm_noalloc_dev(self.handle, C.c_void_p(x.data_ptr()), batch, C.c_void_p(out.data_ptr()),
                                             _stream()))
        return out

    def dequant(self):
        import torch
        out = torch.empty((self.rows, self.cols), dtype=torch.float32, device="cuda")
        check(lib().frk_hip_dequant_dev(self.handle, C.c_void_p(out.data_ptr()), _stream()))
        return out


class BatchActs:
    """A batch's activations quantized once for any number of matrices (the reference's BatchActs::Q8K):
    frk_hip_batch_acts_create / frk_hip_quantize_batch_acts_dev / frk_hip_batch_acts_release."""

    def __init__(self, max_batch, cols):
        h = C.c_void_p()
        check(lib().frk_hip_batch_acts_create(max_batch, cols, C.byref(h)))
        self.handle, self.max_batch, self.cols, self.batch = h, max_batch, cols, 0

    def quantize(self, x):
        import torch
        assert x.dtype == torch.float32 and x.is_cuda and x.is_contiguous() and x.shape[-1] == self.cols
        batch = x.numel() // self.cols
        check(lib().frk_hip_quantize_batch_acts_dev(self.handle, C.c_void_p(x.data_ptr()), batch, _stream()))
        self.batch = batch
        return self

    def release(self):
        if self.handle:
            check(lib().frk_hip_batch_acts_release(self.handle))
            self.handle = None


def _get_rows_dev(self, ids):
    """The embedding gather on device ids (int32 tensor): [len(ids)][cols] f32."""
    import torch
    assert ids.dtype == torch.int32 and ids.is_cuda and ids.is_contiguous()
    out = torch.empty((ids.numel(), self.cols), dtype=torch.float32, device=ids.device)
    check(lib().frk_hip_get_rows_dev(self.handle, C.c_void_p(ids.data_ptr()), ids.numel(), C.c_void_p(out.data_ptr()),
                                     _stream()))
    return out


def _get_rows_host(self, ids):
    """The embedding gather on host ids, every id checked against the table: numpy [len(ids)][cols] f32."""
    import numpy as np
    ids = np.ascontiguousarray(ids, np.int32)
    out = np.empty((ids.size, self.cols), np.float32)
    check(lib().frk_hip_get_rows(self.handle, _np_ptr(ids), ids.size, _np_ptr(out)))
    return out


Weights.get_rows = _get_rows_dev
Weights.get_rows_host = _get_rows_host


def gemm_pair(w0, w1, x, outs=None):
    """frk_hip_gemm_pair_dev: (x W0^T, x W1^T) over one quantization of the batch x[batch][cols]."""
    import torch
    assert x.dtype == torch.float32 and x.is_cuda and x.is_contiguous() and x.shape[-1] == w0.cols == w1.cols
    batch = x.numel() // w0.cols
    y0, y1 = outs if outs is not None else (torch.empty((batch, w.rows), dtype=torch.float32, device=x.device) for w in (w0, w1))
    check(lib().frk_hip_gemm_pair_dev(w0.handle, w1.handle, C.c_void_p(x.data_ptr()), batch, C.c_void_p(y0.data_ptr()),
                                      C.c_void_p(y1.data_ptr()), _stream()))
    return y0, y1


def quantize_q8_k(x):
    """quantize_activations_q8_k on the device: returns (q int8[n], d f32[n/256], bsums int16[n/16])."""
    import torch
    x = x.contiguous()
    n = x.numel()
    q = torch.empty(n, dtype=torch.int8, device=x.device)
    d = torch.empty(n // 256, dtype=torch.float32, device=x.device)
    bs = torch.empty(n // 16, dtype=torch.int16, device=x.device)
    check(lib().frk_hip_quantize_q8_k_dev(C.c_void_p(x.data_ptr()), n, C.c_void_p(q.data_ptr()),
                                          C.c_void_p(d.data_ptr()), C.c_void_p(bs.data_ptr()), _stream()))
    return q, d, bs


def quantize_q8_0(x):
    """quantize_activations_q8 (Avx form) on the device: returns (q int8[n], d f32[n/32])."""
    import torch
    x = x.contiguous()
    n = x.numel()
    q = torch.empty(n, dtype=torch.int8, device=x.device)
    d = torch.empty(n // 32, dtype=torch.float32, device=x.device)
    check(lib().frk_hip_quantize_q8_0_dev(C.c_void_p(x.data_ptr()), n, C.c_void_p(q.data_ptr()),
                                          C.c_void_p(d.data_ptr()), _stream()))
    return q, d


def route_top_k_softmax(logits, k, norm):
    """frink_moe::route_top_k_softmax per row of logits[batch][n_experts]: (ids int32[batch][k], weights f32[batch][k])."""
    import torch
    logits = logits.contiguous()
    batch, n_experts = logits.shape
    ids = torch.empty((batch, k), dtype=torch.int32, device=logits.device)
    w = torch.empty((batch, k), dtype=torch.float32, device=logits.device)
    check(lib().frk_hip_route_top_k_softmax_dev(C.c_void_p(logits.data_ptr()), batch, n_experts, k, int(bool(norm)),
                                                C.c_void_p(ids.data_ptr()), C.c_void_p(w.data_ptr()), _stream()))
    return ids, w


def moe_ffn(gate, up, down, n_experts, x, ids, weights, out=None):
    """Decoder::moe_ffn_batch over experts stacked row-wise in three Weights: x[batch][hidden],
    ids/weights[batch][k] -> out[batch][hidden]."""
    import torch
    assert x.dtype == torch.float32 and x.is_cuda and x.is_contiguous()
    assert ids.dtype == torch.int32 and ids.is_contiguous() and weights.dtype == torch.float32 and weights.is_contiguous()
    batch, k = ids.shape
    y = out if out is not None else torch.empty((batch, down.rows // n_experts), dtype=torch.float32, device=x.device)
    check(lib().frk_hip_moe_ffn_dev(gate.handle, up.handle, down.handle, n_experts, C.c_void_p(x.data_ptr()), batch,
                                    C.c_void_p(ids.data_ptr()), C.c_void_p(weights.data_ptr()), k,
                                    C.c_void_p(y.data_ptr()), _stream()))
    return y


def gemm_grouped(stacked, n_groups, group_off, x, gather=None, out=None):
    """The grouped (indexed) GEMM: pair p of group g (group_off[g] <= p < group_off[g+1]) is row gather[p] of x
    (row p without a gather list) times group g's matrix, rows [g*R, (g+1)*R) of `stacked`; out[pairs][R]."""
    import torch
    assert x.dtype == torch.float32 and x.is_cuda and x.is_contiguous() and x.shape[-1] == stacked.cols
    assert group_off.dtype == torch.int32 and group_off.is_cuda and group_off.numel() == n_groups + 1
    x_rows = x.numel() // stacked.cols
    if gather is not None:
        assert gather.dtype == torch.int32 and gather.is_cuda and gather.is_contiguous()
        pairs = gather.numel()
    else:
        pairs = x_rows
    y = out if out is not None else torch.empty((pairs, stacked.rows // n_groups), dtype=torch.float32, device=x.device)
    check(lib().frk_hip_gemm_grouped_dev(stacked.handle, n_groups, C.c_void_p(group_off.data_ptr()),
                                         C.c_void_p(gather.data_ptr()) if gather is not None else None,
                                         C.c_void_p(x.data_ptr()), x_rows, pairs, C.c_void_p(y.data_ptr()), _stream()))
    return y


# batches of at most this many tokens run per (token, slot) pair on the decode kernels (frk_internal.hpp)
MOE_PER_TOKEN_MAX_BATCH = 16


def moe_intermediates(batch, k, n_experts, hidden, ffn):
    """Test hook: (gate_out, up_out, act_q, act_d, pos_of) of the last moe_ffn call of this shape."""
    import torch
    pairs = batch * k
    g = torch.empty((pairs, ffn), dtype=torch.float32, device="cuda")
    u = torch.empty((pairs, ffn), dtype=torch.float32, device="cuda")
    q = torch.empty((pairs, ffn), dtype=torch.int8, device="cuda")
    d = torch.empty((pairs, ffn // 256), dtype=torch.float32, device="cuda")
    pos = torch.empty((batch, k), dtype=torch.int32, device="cuda")
    check(lib().frk_hip_moe_intermediates_dev(batch, k, n_experts, hidden, ffn, *(C.c_void_p(t.data_ptr())
                                              for t in (g, u, q, d, pos)), _stream()))
    return g, u, q, d, pos


def gemv_multi(ws, x, outs=None):
    """WeightMatrix::apply_gpu_multi on the device: matrices of equal column count share one
    activation (and one Q8_K quantization of it)."""
    import torch
    n = len(ws)
    ys = outs if outs is not None else [torch.empty(w.rows, dtype=torch.float32, device=x.device) for w in ws]
    hs = (C.c_void_p * n)(*[w.handle for w in ws])
    ps = (C.c_void_p * n)(*[y.data_ptr() for y in ys])
    check(lib().frk_hip_gemv_multi_dev(hs, n, C.c_void_p(x.data_ptr()), ps, _stream()))
    return ys


def ffn_swiglu(gate, up, down, x, out=None):
    """down(silu(gate x) * up x), all on the device."""
    import torch
    y = out if out is not None else torch.empty(down.rows, dtype=torch.float32, device=x.device)
    check(lib().frk_hip_ffn_swiglu_dev(gate.handle, up.handle, down.handle, C.c_void_p(x.data_ptr()),
                                       C.c_void_p(y.data_ptr()), _stream()))
    return y


class MatvecLaunch(C.Structure):
    _fields_ = [("kind", C.c_int), ("weights", C.c_void_p), ("weights_len", C.c_size_t), ("rows", C.c_size_t),
                ("row_bytes", C.c_size_t)]

    @classmethod
    def of(cls, kind, weights, rows, row_bytes):
        weights = np.ascontiguousarray(weights, np.uint8)
        m = cls(kind, weights.ctypes.data, weights.size, rows, row_bytes)
        m._keep = weights
        return m


def launch_matvec_multi(x, launches):
    """frink_cuda::matvec_launch::launch_matvec_multi over host buffers."""
    x = np.ascontiguousarray(x, np.float32)
    n = len(launches)
    arr = (MatvecLaunch * n)(*launches)
    outs = [np.empty(l.rows, np.float32) for l in launches]
    ps = (C.c_void_p * n)(*[o.ctypes.data for o in outs])
    check(lib().frk_hip_launch_matvec_multi(_np_ptr(x), x.size, arr, n, ps))
    return outs


def launch_dense_ffn_swiglu(gate, up, down, x):
    """frink_cuda::matvec_launch::launch_dense_ffn_swiglu over host buffers."""
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(down.rows, np.float32)
    check(lib().frk_hip_launch_dense_ffn_swiglu(C.byref(gate), C.byref(up), C.byref(down), _np_ptr(x), x.size,
                                                _np_ptr(out)))
    return out


# ---- host-buffer entry points: numpy in, numpy out ----

def launch_matvec(kind, weights, x, rows, row_bytes):
    """BackendDispatch::launch_matvec: None when the backend has no kernel for `kind`
    (the reference's `None`), raises BackendError when the launch fails (`Some(Err)`)."""
    if not lib().frk_hip_has_launch(kind):
        return None
    weights = np.ascontiguousarray(weights, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(rows, np.float32)
    check(lib().frk_hip_launch_matvec(kind, _np_ptr(weights), weights.size, _np_ptr(x), x.size, rows, row_bytes,
                                      _np_ptr(out)))
    return out


def launch_mul_mm(kind, weights, x_batch, n_rows, n_cols, batch, row_bytes):
    """frink_cuda::mul_mm_launch::launch_mul_mm: out[token*n_rows + row]."""
    weights = np.ascontiguousarray(weights, np.uint8)
    x_batch = np.ascontiguousarray(x_batch, np.float32)
    out = np.empty((batch, n_rows), np.float32)
    check(lib().frk_hip_launch_mul_mm(kind, _np_ptr(weights), weights.size, _np_ptr(x_batch), x_batch.size, n_rows,
                                      n_cols, batch, row_bytes, _np_ptr(out)))
    return out

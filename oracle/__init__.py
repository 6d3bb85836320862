"""ctypes binding of the CPU oracle (``libfrink_oracle.so``).

TEST INFRASTRUCTURE ONLY.  Importable from ``tests/``, from
``__graft_entry__.smoke()`` and from ``bench.py``'s CPU-baseline leg, as the
checker and the timed baseline.  The shipped package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfrink_oracle.so")

Q4_0, Q8_0, Q4_K, Q5_K, Q6_K = 2, 8, 12, 13, 14
Q5_0, IQ4_XS, MXFP4 = 6, 23, 39  # (dequantizers and f32 dots only)
FORM_NEON, FORM_AVX, FORM_SCALAR = 0, 1, 2
F32_DOT, INT_DOT = 0, 1

BLOCK = {Q4_0: (18, 32), Q8_0: (34, 32), Q4_K: (144, 256), Q5_K: (176, 256), Q6_K: (210, 256),
         Q5_0: (22, 32), IQ4_XS: (136, 256), MXFP4: (17, 32)}


def build(force=False):
    """Compile the oracle with gcc (the Makefile beside this file)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        u8p, f32p, i8p, i16p, i32p = (C.POINTER(C.c_uint8), C.POINTER(C.c_float), C.POINTER(C.c_int8),
                                      C.POINTER(C.c_int16), C.POINTER(C.c_int32))
        sz = C.c_size_t
        sig = {
            "fo_f16_to_f32": (C.c_float, [C.c_uint16]),
            "fo_f32_to_f16": (C.c_uint16, [C.c_float]),
            "fo_dequant": (C.c_int, [C.c_int, u8p, sz, f32p]),
            "fo_q4_k_element": (C.c_float, [u8p, C.c_int]),
            "fo_q5_k_element": (C.c_float, [u8p, C.c_int]),
            "fo_q6_k_element": (C.c_float, [u8p, C.c_int]),
            "fo_dot_q8_0_f32": (C.c_float, [u8p, sz, f32p]),
            "fo_dot_q4_0_f32": (C.c_float, [u8p, sz, f32p]),
            "fo_dot_q4_k_f32": (C.c_float, [u8p, sz, f32p]),
            "fo_dot_q5_k_f32": (C.c_float, [u8p, sz, f32p]),
            "fo_dot_q6_k_f32": (C.c_float, [u8p, sz, f32p]),
            "fo_dot_q5_0_f32": (C.c_float, [u8p, sz, f32p]),
            "fo_dot_iq4_xs_f32": (C.c_float, [u8p, sz, f32p]),
            "fo_dot_mxfp4_f32": (C.c_float, [u8p, sz, f32p]),
            "fo_quantize_q8_k": (None, [f32p, sz, i8p, f32p, i16p]),
            "fo_quantize_q8_0": (None, [f32p, sz, C.c_int, i8p, f32p]),
            "fo_dot_q8_0_q8": (C.c_float, [u8p, sz, i8p, f32p]),
            "fo_dot_q4_0_q8": (C.c_float, [u8p, sz, i8p, f32p]),
            "fo_dot_q5_0_q8": (C.c_float, [u8p, sz, i8p, f32p]),
            "fo_dot_mxfp4_q8": (C.c_float, [u8p, sz, i8p, f32p]),
            "fo_dot_iq4_xs_q8k": (C.c_float, [u8p, sz, i8p, f32p]),
            "fo_decode_q5_0_block": (None, [u8p, i8p]),
            "fo_decode_mxfp4_block": (None, [u8p, i8p]),
            "fo_e8m0_half_scale": (C.c_float, [C.c_uint8]),
            "fo_dot_q4_k_q8k": (C.c_float, [u8p, sz, i8p, f32p, i16p]),
            "fo_dot_q5_k_q8k": (C.c_float, [u8p, sz, i8p, f32p, i16p]),
            "fo_dot_q6_k_q8k": (C.c_float, [u8p, sz, i8p, f32p]),
            "fo_nearest_int": (C.c_int, [C.c_float]),
            "fo_make_qx_quants": (C.c_float, [C.c_int, C.c_int, f32p, i8p, C.c_int]),
            "fo_encode_row_q8_0": (C.c_int, [f32p, sz, u8p]),
            "fo_encode_row_q4_k": (C.c_int, [f32p, sz, u8p]),
            "fo_encode_row_q5_k": (C.c_int, [f32p, sz, u8p]),
            "fo_encode_row_q6_k": (C.c_int, [f32p, sz, u8p]),
            "fo_encode_matrix": (C.c_int, [C.c_int, f32p, sz, sz, u8p, C.c_int]),
            "fo_gemm": (C.c_int, [C.c_int, u8p, sz, sz, f32p, sz, f32p, C.c_int, C.c_int]),
            "fo_gemm_rows": (C.c_int, [C.c_int, u8p, sz, sz, sz, sz, f32p, sz, f32p, C.c_int, C.c_int]),
            "fo_silu": (C.c_float, [C.c_float]),
            "fo_swiglu": (None, [f32p, f32p, sz, f32p]),
            "fo_route_top_k_softmax": (None, [f32p, C.c_int, C.c_int, C.c_int, i32p, f32p]),
            "fo_moe_ffn_batch": (C.c_int, [C.c_int, u8p, u8p, u8p, C.c_int, C.c_int, C.c_int, f32p,
                                           C.c_int, i32p, f32p, C.c_int, f32p, C.c_int]),
            "fo_moe_ffn_per_position": (C.c_int, [C.c_int, u8p, u8p, u8p, C.c_int, C.c_int, C.c_int, f32p,
                                                  C.c_int, i32p, f32p, C.c_int, f32p, C.c_int]),
            "fo_have_avx2": (C.c_int, []),
            "fo_e8m0_scale": (C.c_float, [C.c_uint8]),
            "fo_avx2_gemv_q4_k_f32": (C.c_int, [u8p, sz, sz, f32p, f32p, C.c_int]),
            "fo_avx2_gemm_q4_k_q8k": (C.c_int, [u8p, sz, sz, f32p, sz, f32p, C.c_int]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(C.POINTER(ct))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    if isinstance(a, (bytes, bytearray)):
        a = np.frombuffer(bytes(a), dtype=np.uint8)
    return np.ascontiguousarray(a, dtype=np.uint8)


def f16_to_f32(h):
    return lib().fo_f16_to_f32(int(h))


def f32_to_f16(f):
    return lib().fo_f32_to_f16(float(np.float32(f)))


def dequant(kind, data):
    data = _u8(data)
    bb, be = BLOCK[kind]
    out = np.empty(data.size // bb * be, dtype=np.float32)
    rc = lib().fo_dequant(kind, _p(data, C.c_uint8), data.size, _p(out, C.c_float))
    if rc:
        raise ValueError("buffer length %d is not a multiple of the block size %d" % (data.size, bb))
    return out


def element(kind, block, i):
    block = _u8(block)
    fn = {Q4_K: lib().fo_q4_k_element, Q5_K: lib().fo_q5_k_element, Q6_K: lib().fo_q6_k_element}[kind]
    return fn(_p(block, C.c_uint8), i)


def dot_f32(kind, row, x):
    row, x = _u8(row), _f32(x)
    fn = {Q4_0: lib().fo_dot_q4_0_f32, Q8_0: lib().fo_dot_q8_0_f32, Q4_K: lib().fo_dot_q4_k_f32, Q5_K: lib().fo_dot_q5_k_f32,
          Q6_K: lib().fo_dot_q6_k_f32, Q5_0: lib().fo_dot_q5_0_f32, IQ4_XS: lib().fo_dot_iq4_xs_f32,
          MXFP4: lib().fo_dot_mxfp4_f32}[kind]
    return fn(_p(row, C.c_uint8), row.size, _p(x, C.c_float))


def quantize_q8_k(x):
    x = _f32(x).ravel()
    nb = x.size // 256
    q = np.empty(nb * 256, np.int8)
    d = np.empty(nb, np.float32)
    bs = np.empty(nb * 16, np.int16)
    lib().fo_quantize_q8_k(_p(x, C.c_float), x.size, _p(q, C.c_int8), _p(d, C.c_float), _p(bs, C.c_int16))
    return q, d, bs


def quantize_q8_0(x, form=FORM_AVX):
    x = _f32(x).ravel()
    nb = x.size // 32
    q = np.empty(nb * 32, np.int8)
    d = np.empty(nb, np.float32)
    lib().fo_quantize_q8_0(_p(x, C.c_float), x.size, form, _p(q, C.c_int8), _p(d, C.c_float))
    return q, d


def dot_int(kind, row, acts):
    row = _u8(row)
    if kind in (Q8_0, Q4_0, Q5_0, MXFP4):
        q, d = acts
        fn = {Q8_0: lib().fo_dot_q8_0_q8, Q4_0: lib().fo_dot_q4_0_q8, Q5_0: lib().fo_dot_q5_0_q8,
              MXFP4: lib().fo_dot_mxfp4_q8}[kind]
        return fn(_p(row, C.c_uint8), row.size, _p(q, C.c_int8), _p(d, C.c_float))
    q, d, bs = acts
    if kind == IQ4_XS:
        return lib().fo_dot_iq4_xs_q8k(_p(row, C.c_uint8), row.size, _p(q, C.c_int8), _p(d, C.c_float))
    if kind in (Q4_K, Q5_K):
        fn = lib().fo_dot_q4_k_q8k if kind == Q4_K else lib().fo_dot_q5_k_q8k
        return fn(_p(row, C.c_uint8), row.size, _p(q, C.c_int8), _p(d, C.c_float), _p(bs, C.c_int16))
    return lib().fo_dot_q6_k_q8k(_p(row, C.c_uint8), row.size, _p(q, C.c_int8), _p(d, C.c_float))


def nearest_int(f):
    return lib().fo_nearest_int(float(np.float32(f)))


def make_qx_quants(x, nmax=32, rmse_type=1):
    x = _f32(x)
    l = np.full(x.size, 7, np.int8)
    s = lib().fo_make_qx_quants(x.size, nmax, _p(x, C.c_float), _p(l, C.c_int8), rmse_type)
    return s, l


def encode_row(kind, x):
    """Returns the block bytes, or None when the length is not a whole number of blocks."""
    x = _f32(x).ravel()
    bb, be = BLOCK[kind]
    out = np.empty(x.size // be * bb, np.uint8)
    fn = {Q8_0: lib().fo_encode_row_q8_0, Q4_K: lib().fo_encode_row_q4_k, Q5_K: lib().fo_encode_row_q5_k,
          Q6_K: lib().fo_encode_row_q6_k}[kind]
    if fn(_p(x, C.c_float), x.size, _p(out, C.c_uint8)):
        return None
    return out


def encode_matrix(kind, w, threads=0):
    w = _f32(w)
    rows, cols = w.shape
    bb, be = BLOCK[kind]
    out = np.empty(rows * (cols // be) * bb, np.uint8)
    rc = lib().fo_encode_matrix(kind, _p(w, C.c_float), rows, cols, _p(out, C.c_uint8), threads)
    if rc == -2:
        raise ValueError("quant kind %d has no encoder here" % kind)
    if rc:
        raise ValueError("cols %d is not a whole number of %d-element blocks" % (cols, be))
    return out


def gemm(kind, w, rows, cols, x, mode=INT_DOT, threads=0, row0=0, nrows=None):
    """x: [batch][cols] -> [batch][nrows]"""
    w, x = _u8(w), _f32(x).reshape(-1, cols)
    batch = x.shape[0]
    nrows = rows - row0 if nrows is None else nrows
    y = np.empty((batch, nrows), np.float32)
    rc = lib().fo_gemm_rows(kind, _p(w, C.c_uint8), rows, cols, row0, nrows, _p(x, C.c_float), batch,
                            _p(y, C.c_float), mode, threads)
    if rc:
        raise ValueError("fo_gemm_rows rc=%d" % rc)
    return y


def gemv(kind, w, rows, cols, x, mode=INT_DOT, threads=0):
    return gemm(kind, w, rows, cols, _f32(x).reshape(1, cols), mode, threads)[0]


def silu(x):
    return lib().fo_silu(float(np.float32(x)))


def swiglu(g, u):
    g, u = _f32(g).ravel(), _f32(u).ravel()
    out = np.empty_like(g)
    lib().fo_swiglu(_p(g, C.c_float), _p(u, C.c_float), g.size, _p(out, C.c_float))
    return out


def route_top_k_softmax(logits, k, norm_topk_prob=True):
    logits = _f32(logits).ravel()
    k = min(k, logits.size)
    ids = np.empty(k, np.int32)
    w = np.empty(k, np.float32)
    lib().fo_route_top_k_softmax(_p(logits, C.c_float), logits.size, k, int(norm_topk_prob),
                                 _p(ids, C.c_int32), _p(w, C.c_float))
    return ids, w


MOE_BUCKET_FROM = 32  # ffn_batch.rs:355: smaller batches run per position


def moe_ffn(kind, gate, up, down, n_experts, hidden, ffn, x, ids, weights, threads=0):
    """The MoE layer the way the reference runs a batch of this size: bucketed by expert from 32
    tokens on (experts added in ascending id), per position below (slots added in routing order)."""
    batch = _f32(x).reshape(-1, hidden).shape[0]
    fn = moe_ffn_batch if batch >= MOE_BUCKET_FROM else moe_ffn_per_position
    return fn(kind, gate, up, down, n_experts, hidden, ffn, x, ids, weights, threads)


def moe_ffn_per_position(kind, gate, up, down, n_experts, hidden, ffn, x, ids, weights, threads=0):
    return moe_ffn_batch(kind, gate, up, down, n_experts, hidden, ffn, x, ids, weights, threads,
                         _fn="fo_moe_ffn_per_position")


def moe_ffn_batch(kind, gate, up, down, n_experts, hidden, ffn, x, ids, weights, threads=0, _fn="fo_moe_ffn_batch"):
    gate, up, down = _u8(gate), _u8(up), _u8(down)
    x = _f32(x).reshape(-1, hidden)
    batch = x.shape[0]
    ids = np.ascontiguousarray(ids, np.int32).reshape(batch, -1)
    weights = _f32(weights).reshape(batch, -1)
    k = ids.shape[1]
    out = np.empty((batch, hidden), np.float32)
    rc = getattr(lib(), _fn)(kind, _p(gate, C.c_uint8), _p(up, C.c_uint8), _p(down, C.c_uint8),
                                n_experts, hidden, ffn, _p(x, C.c_float), batch, _p(ids, C.c_int32),
                                _p(weights, C.c_float), k, _p(out, C.c_float), threads)
    if rc:
        raise ValueError("%s rc=%d" % (_fn, rc))
    return out


def have_avx2():
    return bool(lib().fo_have_avx2())


def avx2_gemv_q4_k_f32(w, rows, cols, x, threads=1):
    """The reference's x86 decode default (AVX2+FMA f32 dot), for the timed CPU baseline."""
    w, x = _u8(w), _f32(x).ravel()
    y = np.empty(rows, np.float32)
    rc = lib().fo_avx2_gemv_q4_k_f32(_p(w, C.c_uint8), rows, cols, _p(x, C.c_float), _p(y, C.c_float), threads)
    if rc:
        raise RuntimeError("fo_avx2_gemv_q4_k_f32 rc=%d (no AVX2+FMA on this host?)" % rc)
    return y


def avx2_gemm_q4_k_q8k(w, rows, cols, x, threads=1):
    """x: [batch][cols] -> [batch][rows]: Q8_K quantization + AVX2 integer dots, weight row outermost."""
    w, x = _u8(w), _f32(x).reshape(-1, cols)
    y = np.empty((x.shape[0], rows), np.float32)
    rc = lib().fo_avx2_gemm_q4_k_q8k(_p(w, C.c_uint8), rows, cols, _p(x, C.c_float), x.shape[0], _p(y, C.c_float), threads)
    if rc:
        raise RuntimeError("fo_avx2_gemm_q4_k_q8k rc=%d (no AVX2+FMA on this host?)" % rc)
    return y

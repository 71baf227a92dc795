"""TEST INFRASTRUCTURE ONLY: numpy-facing binding of the CPU checker (oracle/liboracle.so).

May be imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py,
always as the checker and never as the thing measured or shipped.  The arithmetic and the
reference lines it follows are documented in oracle/oracle.c.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# CN_ORACLE_LIB names another build of the same sources (the sanitizer build, oracle/_asan/liboracle.so)
_SO = os.environ.get("CN_ORACLE_LIB") or os.path.join(_HERE, "liboracle.so")

_c = ctypes
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
_i64p = np.ctypeslib.ndpointer(np.int64, flags="C_CONTIGUOUS")


def build():
    """Compile oracle/liboracle.so with the committed Makefile."""
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def _load():
    if not os.path.exists(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    lib.cn_oracle_table.argtypes = [_f32p]
    for name in ("cn_oracle_compress_literal", "cn_oracle_compress_closed"):
        getattr(lib, name).argtypes = [_f32p, _c.c_float, _c.c_size_t, _u8p, _c.c_int]
    lib.cn_oracle_decode_lut.argtypes = [_c.c_float, _f32p]
    lib.cn_oracle_decompress.argtypes = [_u8p, _c.c_float, _c.c_size_t, _f32p]
    lib.cn_oracle_decompress_axpy.argtypes = [_u8p, _c.c_float, _c.c_float, _c.c_size_t, _f32p]
    lib.cn_oracle_rmsprop_update.argtypes = [_f32p, _f32p, _f32p, _c.c_float, _c.c_float, _c.c_size_t]
    _i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
    lib.cn_oracle_csr_from_dense.argtypes = [_f32p, _c.c_int64, _c.c_int64, _c.c_int, _i32p, _c.c_void_p, _c.c_void_p]
    lib.cn_oracle_csr_from_dense.restype = _c.c_int64
    lib.cn_oracle_csr_gemm.argtypes = [_c.c_int64, _c.c_int64, _i32p, _i32p, _f32p, _f32p, _f32p]
    lib.cn_oracle_absmax.argtypes = [_f32p, _c.c_size_t]
    lib.cn_oracle_absmax.restype = _c.c_float
    g = [_c.c_int, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _f32p, _c.c_int64, _f32p,
         _c.c_int64, _f32p, _c.c_int64]
    lib.cn_oracle_gemm_f64acc.argtypes = g
    lib.cn_oracle_gemm_f32_seqfma.argtypes = g
    lib.cn_oracle_gemm_f64acc_abs.argtypes = [_c.c_int, _c.c_int, _c.c_int64, _c.c_int64,
                                              _c.c_int64, _f32p, _c.c_int64, _f32p, _c.c_int64,
                                              _f64p, _f64p]
    lib.cn_oracle_gemm_cols_f64acc.argtypes = [_c.c_int, _c.c_int, _c.c_int64, _c.c_int64, _f32p,
                                               _c.c_int64, _f32p, _c.c_int64, _i64p, _c.c_int64,
                                               _f64p, _f64p]
    lib.cn_oracle_gemm_w8_f64acc.argtypes = [_c.c_int64, _c.c_int64, _c.c_int64, _f32p,
                                             _c.c_int64, _u8p, _c.c_int64, _c.c_float, _f32p,
                                             _c.c_int64]
    lib.cn_oracle_dot8bit_tables.argtypes = [_c.c_float, _c.c_float, _f32p, _f32p]
    lib.cn_oracle_dot8bit.argtypes = [_u8p, _u8p, _f32p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_float, _c.c_float,
                                      _c.c_void_p]
    lib.cn_oracle_add_row_vector.argtypes = [_f32p, _f32p, _c.c_int64, _c.c_int64, _f32p]
    lib.cn_oracle_maxout.argtypes = [_f32p, _c.c_int64, _c.c_int64, _c.c_int, _f32p, _f32p]
    lib.cn_oracle_expand_to_maxout_grad.argtypes = [_f32p, _f32p, _c.c_int64, _c.c_int64,
                                                    _c.c_int, _f32p]
    lib.cn_oracle_softmax.argtypes = [_f32p, _c.c_int64, _c.c_int64, _f32p]
    lib.cn_oracle_num_threads.restype = _c.c_int
    lib.cn_oracle_set_threads.argtypes = [_c.c_int]
    lib.cn_port_compress.argtypes = [_f32p, _c.c_float, _c.c_size_t, _u8p]
    lib.cn_port_decompress.argtypes = [_u8p, _c.c_float, _c.c_size_t, _f32p]
    lib.cn_port_absmax.argtypes = [_f32p, _c.c_size_t]
    lib.cn_port_absmax.restype = _c.c_float
    lib.cn_port_gemm_nn.argtypes = [_c.c_int64, _c.c_int64, _c.c_int64, _f32p, _c.c_int64, _f32p,
                                    _c.c_int64, _f32p, _c.c_int64]
    lib.cn_port_gemm.argtypes = [_c.c_int, _c.c_int, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_int64,
                                 _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int64]
    return lib


_lib = _load()


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def table():
    t = np.empty(126, np.float32)
    _lib.cn_oracle_table(t)
    return t


def compress(x, precision, sliver_rule=0, form="literal"):
    x = _f32(x)
    out = np.empty(x.shape, np.uint8)
    fn = _lib.cn_oracle_compress_literal if form == "literal" else _lib.cn_oracle_compress_closed
    fn(x.reshape(-1), float(precision), x.size, out.reshape(-1), int(sliver_rule))
    return out


def decode_lut(precision):
    lut = np.empty(256, np.float32)
    _lib.cn_oracle_decode_lut(float(precision), lut)
    return lut


def decompress(codes, precision):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape, np.float32)
    _lib.cn_oracle_decompress(codes.reshape(-1), float(precision), codes.size, out.reshape(-1))
    return out


def decompress_axpy(codes, precision, alpha, y):
    """Returns y + alpha * decode(codes) (y is not modified)."""
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.array(y, dtype=np.float32, order="C", copy=True)
    _lib.cn_oracle_decompress_axpy(codes.reshape(-1), float(precision), float(alpha), codes.size, out.reshape(-1))
    return out


def rmsprop_update(rms, grad, w, rms_multiplier, learning_rate):
    """Returns (rms', w') of one RMSprop-with-weight-update pass (inputs are not modified)."""
    r = np.array(rms, dtype=np.float32, order="C", copy=True)
    ww = np.array(w, dtype=np.float32, order="C", copy=True)
    g = _f32(grad)
    _lib.cn_oracle_rmsprop_update(r.reshape(-1), g.reshape(-1), ww.reshape(-1), float(rms_multiplier),
                                  float(learning_rate), g.size)
    return r, ww


def csr_from_dense(A, transpose=False):
    """(row_ptr, col_idx, vals) of A, or of A^T when `transpose`."""
    A = _f32(A)
    rows, cols = A.shape
    R = cols if transpose else rows
    row_ptr = np.zeros(R + 1, np.int32)
    nnz = _lib.cn_oracle_csr_from_dense(A, rows, cols, int(transpose), row_ptr, None, None)
    col_idx = np.zeros(max(nnz, 1), np.int32)
    vals = np.zeros(max(nnz, 1), np.float32)
    _lib.cn_oracle_csr_from_dense(A, rows, cols, int(transpose), row_ptr, col_idx.ctypes.data, vals.ctypes.data)
    return row_ptr, col_idx[:nnz], vals[:nnz]


def _csr_arrays(csr):
    row_ptr, col_idx, vals = csr
    pad = lambda a, t: np.ascontiguousarray(a if a.size else np.zeros(1, t), t)
    return np.ascontiguousarray(row_ptr, np.int32), pad(col_idx, np.int32), pad(vals, np.float32)


def csr_gemm(csr, B):
    """S B for S = (row_ptr, col_idx, vals)."""
    row_ptr, col_idx, vals = _csr_arrays(csr)
    B = _f32(B)
    out = np.empty((row_ptr.size - 1, B.shape[1]), np.float32)
    _lib.cn_oracle_csr_gemm(row_ptr.size - 1, B.shape[1], row_ptr, col_idx, vals, B, out)
    return out


def absmax(x):
    x = _f32(x)
    return float(_lib.cn_oracle_absmax(x.reshape(-1), x.size))


def _gemm_dims(A, B, ta, tb):
    M, K = (A.shape[1], A.shape[0]) if ta else A.shape
    K2, N = (B.shape[1], B.shape[0]) if tb else B.shape
    if K != K2:
        raise ValueError("inner dimensions differ: %d vs %d" % (K, K2))
    return M, N, K


def gemm(A, B, ta=False, tb=False, mode="f64acc"):
    """C = op(A) op(B) on row-major arrays; mode 'f64acc' (yard-stick) or 'seqfma'."""
    A, B = _f32(A), _f32(B)
    M, N, K = _gemm_dims(A, B, ta, tb)
    C = np.empty((M, N), np.float32)
    fn = _lib.cn_oracle_gemm_f64acc if mode == "f64acc" else _lib.cn_oracle_gemm_f32_seqfma
    fn(int(ta), int(tb), M, N, K, A, A.shape[1], B, B.shape[1], C, N)
    return C


def gemm_with_abs(A, B, ta=False, tb=False):
    """(C, sum_k |a||b|) in float64."""
    A, B = _f32(A), _f32(B)
    M, N, K = _gemm_dims(A, B, ta, tb)
    C = np.empty((M, N), np.float64)
    Cabs = np.empty((M, N), np.float64)
    _lib.cn_oracle_gemm_f64acc_abs(int(ta), int(tb), M, N, K, A, A.shape[1], B, B.shape[1], C, Cabs)
    return C, Cabs


def gemm_cols(A, B, cols, ta=False, tb=False):
    """Selected output columns, float64: returns (C[:, cols], sum_k|a||b|[:, cols])."""
    A, B = _f32(A), _f32(B)
    M, N, K = _gemm_dims(A, B, ta, tb)
    cols = np.ascontiguousarray(cols, dtype=np.int64)
    C = np.empty((M, cols.size), np.float64)
    Cabs = np.empty((M, cols.size), np.float64)
    _lib.cn_oracle_gemm_cols_f64acc(int(ta), int(tb), M, K, A, A.shape[1], B, B.shape[1], cols,
                                    cols.size, C, Cabs)
    return C, Cabs


def gemm_w8(A, W, scale):
    A = _f32(A)
    W = np.ascontiguousarray(W, dtype=np.uint8)
    M, K = A.shape
    K2, N = W.shape
    if K != K2:
        raise ValueError("inner dimensions differ")
    C = np.empty((M, N), np.float32)
    _lib.cn_oracle_gemm_w8_f64acc(M, N, K, A, K, W, N, float(scale), C, N)
    return C


def dot8bit_tables(precision_a, precision_b):
    ta, tb = np.empty(256, np.float32), np.empty(256, np.float32)
    _lib.cn_oracle_dot8bit_tables(float(precision_a), float(precision_b), ta, tb)
    return ta, tb


def dot8bit(A, B, precision_a, precision_b, out=None):
    """(out + decodeA(A) decodeB(B), sum_k |a||b|): kDot8bit's sum, term by term in fp32, added to `out` (zeros if None)."""
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    M, K = A.shape
    K2, N = B.shape
    if K != K2:
        raise ValueError("inner dimensions differ")
    res = np.zeros((M, N), np.float32) if out is None else np.array(out, dtype=np.float32, order="C")
    mag = np.empty((M, N), np.float64)
    _lib.cn_oracle_dot8bit(A, B, res, M, K, N, float(precision_a), float(precision_b), mag.ctypes.data)
    return res, mag


def add_row_vector(A, v):
    A, v = _f32(A), _f32(v).reshape(-1)
    out = np.empty_like(A)
    _lib.cn_oracle_add_row_vector(A, v, A.shape[0], A.shape[1], out)
    return out


def maxout(A, pool):
    A = _f32(A)
    out = np.empty((A.shape[0], A.shape[1] // pool), np.float32)
    arg = np.empty_like(out)
    _lib.cn_oracle_maxout(A, A.shape[0], A.shape[1], int(pool), out, arg)
    return out, arg


def expand_to_maxout_grad(err, argmax, pool):
    err, argmax = _f32(err), _f32(argmax)
    out = np.empty((err.shape[0], err.shape[1] * pool), np.float32)
    _lib.cn_oracle_expand_to_maxout_grad(err, argmax, err.shape[0], err.shape[1], int(pool), out)
    return out


def softmax(A):
    A = _f32(A)
    out = np.empty_like(A)
    _lib.cn_oracle_softmax(A, A.shape[0], A.shape[1], out)
    return out


def num_threads():
    return int(_lib.cn_oracle_num_threads())


def set_threads(n):
    _lib.cn_oracle_set_threads(int(n))


def port_compress(x, precision):
    x = _f32(x)
    out = np.empty(x.shape, np.uint8)
    _lib.cn_port_compress(x.reshape(-1), float(precision), x.size, out.reshape(-1))
    return out


def port_decompress(codes, precision):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape, np.float32)
    _lib.cn_port_decompress(codes.reshape(-1), float(precision), codes.size, out.reshape(-1))
    return out


def port_absmax(x):
    x = _f32(x)
    return float(_lib.cn_port_absmax(x.reshape(-1), x.size))


def port_gemm_nn(A, B):
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    K2, N = B.shape
    if K != K2:
        raise ValueError("inner dimensions differ")
    C = np.empty((M, N), np.float32)
    _lib.cn_port_gemm_nn(M, N, K, A, K, B, N, C, N)
    return C


def port_gemm(A, B, ta=False, tb=False, out=None, accumulate=False, lda=None):
    """out (+)= op(A) op(B) on all OpenMP threads, fp32 accumulation; `lda` lets A be a column block of a wider
    row-major matrix (pass the block as a view, its leading dimension here)."""
    M, K = (A.shape[1], A.shape[0]) if ta else A.shape
    K2, N = (B.shape[1], B.shape[0]) if tb else B.shape
    if K != K2:
        raise ValueError("inner dimensions differ")
    B = _f32(B)
    if lda is None:
        A = _f32(A)
        lda = A.shape[1]
    elif A.dtype != np.float32 or A.strides[1] != 4 or A.strides[0] != 4 * lda:
        raise ValueError("A is not a float32 block with leading dimension %d" % lda)
    if out is None:
        out = np.empty((M, N), np.float32)
        accumulate = False
    _lib.cn_port_gemm(int(ta), int(tb), int(accumulate), M, N, K, A.ctypes.data, lda, B.ctypes.data, B.shape[1],
                      out.ctypes.data, N)
    return out

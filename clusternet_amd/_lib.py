"""ctypes binding of libcnhip.so.  No computation happens here and there is no CPU fallback: if
the library is missing or no GPU is usable, calls raise."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# CNHIP_LIB names another build of the same library (the host-sanitizer build of `python -m clusternet_amd.build
# --host-asan`); CNHIP_NO_TORCH=1 keeps a host-only process from loading PyTorch first.
_PATH = os.environ.get("CNHIP_LIB") or os.path.join(_HERE, "libcnhip.so")
_lib = None


class CnError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("libcnhip status %d: %s" % (status, message))
        self.status = status


def lib_path():
    return _PATH


def lib():
    """Loads libcnhip.so (after torch, so that both share one HIP runtime)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_PATH):
        raise ImportError("%s is not built; run `python -m clusternet_amd.build`" % _PATH)
    if not os.environ.get("CNHIP_NO_TORCH"):
        try:
            import torch  # noqa: F401  (loads the HIP runtime that owns the tensors we are handed)
        except ImportError:
            pass
    L = C.CDLL(_PATH)
    i64, vp, f32, sz = C.c_int64, C.c_void_p, C.c_float, C.c_size_t
    L.cn_status_string.restype = C.c_char_p
    L.cn_status_string.argtypes = [C.c_int]
    L.cn_last_error.restype = C.c_char_p
    L.cn_init.argtypes = [C.c_int]
    L.cn_num_compute_units.restype = C.c_int
    L.cn_malloc.argtypes = [C.POINTER(vp), sz]
    L.cn_free.argtypes = [vp]
    L.cn_memcpy_h2d.argtypes = [vp, vp, sz]
    L.cn_memcpy_d2h.argtypes = [vp, vp, sz]
    L.cn_memcpy_d2d.argtypes = [vp, vp, sz, vp]
    L.cn_fill_f32.argtypes = [vp, f32, sz, vp]
    L.cn_synchronize.argtypes = [vp]
    L.cn_table_get.argtypes = [C.POINTER(f32)]
    L.cn_gemm_f32.argtypes = [C.c_int, C.c_int, i64, i64, i64, vp, i64, vp, i64, vp, i64, vp]
    L.cn_gemm_f32_noalloc.argtypes = [C.c_int, C.c_int, i64, i64, i64, vp, i64, vp, i64, vp, i64, vp]
    L.cn_gemm_f32_absmax.argtypes = [C.c_int, C.c_int, i64, i64, i64, vp, i64, vp, i64, vp, i64, vp, vp]
    L.cn_gemm_f32_w8.argtypes = [i64, i64, i64, vp, i64, vp, i64, f32, vp, i64, vp]
    L.cn_gemm_c8c8_add.argtypes = [i64, i64, i64, vp, i64, vp, i64, f32, f32, vp, i64, vp]
    L.cn_csr_from_dense_f32.argtypes = [vp, i64, i64, i64, C.c_int, vp, vp, vp, i64, C.POINTER(i64), vp]
    L.cn_csr_gemm_f32.argtypes = [i64, i64, i64, vp, vp, vp, vp, i64, vp, i64, vp]
    L.cn_csr_transpose.argtypes = [i64, i64, i64, vp, vp, vp, vp, vp, vp, vp, vp]
    L.cn_csr_gemm_f32_absmax.argtypes = [i64, i64, i64, vp, vp, vp, vp, i64, vp, i64, vp, vp]
    L.cn_csr_gemm_coded_update.argtypes = [i64, i64, i64, vp, vp, vp, vp, i64, vp, vp, vp, i64, f32, vp]
    L.cn_csr_gemm_coded_rmsprop.argtypes = [i64, i64, i64, vp, vp, vp, vp, i64, vp, vp, vp, vp, i64, f32, f32, vp]
    L.cn_compress_8bit_axpy.argtypes = [vp, f32, sz, vp, f32, vp, vp]
    L.cn_compress_8bit_axpy_dp.argtypes = [vp, vp, sz, vp, f32, vp, vp]
    L.cn_csr_to_dense_f32.argtypes = [i64, i64, vp, vp, vp, vp, i64, vp]
    L.cn_absmax_f32.argtypes = [vp, sz, vp, vp]
    L.cn_compress_8bit.argtypes = [vp, f32, sz, vp, vp]
    L.cn_compress_8bit_dp.argtypes = [vp, vp, sz, vp, vp]
    L.cn_decompress_8bit.argtypes = [vp, f32, sz, vp, vp]
    L.cn_decompress_8bit_dp.argtypes = [vp, vp, sz, vp, vp]
    L.cn_decode_8bit_lut.argtypes = [vp, vp, sz, vp, vp]
    L.cn_absmax_compress_8bit.argtypes = [vp, sz, vp, vp, vp]
    L.cn_host_absmax_compress_single_launch.argtypes = [C.c_int]
    L.cn_host_absmax_compress_single_launch.restype = None
    L.cn_host_absmax_compress_spin_limit.argtypes = [C.c_int]
    L.cn_host_absmax_compress_spin_limit.restype = None
    L.cn_decompress_8bit_axpy.argtypes = [vp, f32, f32, sz, vp, vp]
    L.cn_decompress_8bit_axpy_dp.argtypes = [vp, vp, f32, sz, vp, vp]
    L.cn_rmsprop_update_f32.argtypes = [vp, vp, vp, f32, f32, sz, vp]
    L.cn_rmsprop_update_w8.argtypes = [vp, vp, f32, vp, f32, f32, sz, vp]
    L.cn_rmsprop_update_w8_dp.argtypes = [vp, vp, vp, vp, f32, f32, sz, vp]
    L.cn_host_encode_exact.argtypes = [f32, f32]
    L.cn_host_plan_gemm.argtypes = [i64, i64, i64, C.c_int, sz, C.c_int, C.POINTER(i64)]
    L.cn_host_plan_gemm.restype = None
    L.cn_host_plan_gemm_rows_along_k.argtypes = [i64, i64, i64, C.c_int, sz, C.c_int, C.POINTER(i64)]
    L.cn_host_plan_gemm_rows_along_k.restype = None
    L.cn_host_force_gemm_tile_n.argtypes = [C.c_int]
    L.cn_host_force_gemm_tile_n.restype = None
    L.cn_host_gemm_epilogue_in_kernel.argtypes = [C.c_int]
    L.cn_host_gemm_epilogue_in_kernel.restype = None
    L.cn_host_gemm_wide_store.argtypes = [C.c_int]
    L.cn_host_gemm_wide_store.restype = None
    L.cn_host_codec_encoder.argtypes = [C.c_int]
    L.cn_host_codec_encoder.restype = None
    L.cn_host_quotient_mismatches.argtypes = [C.c_float, C.c_uint32, C.c_ulonglong]
    L.cn_host_quotient_mismatches.restype = C.c_longlong
    L.cn_host_gemm_w8_rows.argtypes = [C.c_int]
    L.cn_host_gemm_w8_rows.restype = None
    L.cn_host_gemm_small.argtypes = [C.c_int]
    L.cn_host_gemm_small.restype = None
    L.cn_host_gemm_persistent.argtypes = [C.c_int]
    L.cn_host_gemm_persistent.restype = None
    L.cn_host_last_gemm_kernel.argtypes = [C.c_void_p]
    L.cn_host_last_gemm_kernel.restype = C.c_int
    L.cn_host_tile_counters_in_use.argtypes = []
    L.cn_host_tile_counters_in_use.restype = C.c_int
    L.cn_host_stream_slots.argtypes = [C.POINTER(C.c_uint64), C.c_int, C.POINTER(C.c_int)]
    L.cn_host_stream_slots.restype = None
    L.cn_host_reduction_fences.argtypes = [C.c_int]
    L.cn_host_reduction_fences.restype = None
    L.cn_host_csr_strip_kernel.argtypes = [C.c_int]
    L.cn_host_csr_strip_kernel.restype = None
    L.cn_host_csr_rows_workgroups_per_cu.argtypes = [C.c_int]
    L.cn_host_csr_rows_workgroups_per_cu.restype = None
    L.cn_host_csr_lds_rows.argtypes = [C.c_int]
    L.cn_host_csr_lds_rows.restype = None
    L.cn_host_csr_paired_rows.argtypes = [C.c_int]
    L.cn_host_csr_paired_rows.restype = None
    _lib = L
    return L


def check(status):
    if status != 0:
        L = lib()
        raise CnError(status, "%s: %s" % (L.cn_status_string(status).decode(), L.cn_last_error().decode()))


def init(device=0):
    check(lib().cn_init(int(device)))


def num_compute_units():
    return int(lib().cn_num_compute_units())


def table():
    import numpy as np
    buf = (C.c_float * 126)()
    check(lib().cn_table_get(buf))
    return np.frombuffer(buf, dtype=np.float32).copy()


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(t, dtype, what):
    import torch
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype):
        raise TypeError("%s must be a CUDA/HIP tensor of dtype %s" % (what, dtype))
    if t.dim() == 2 and t.stride(1) != 1 and t.shape[1] > 1:
        raise ValueError("%s must be row-major (unit column stride)" % what)


def _ld(t):
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)


def gemm(A, B, trans_a=False, trans_b=False, out=None, absmax_out=None, noalloc=False):
    """out = op(A) op(B) on row-major fp32 matrices; mirrors ClusterNet::dot(A,B,out,T1,T2).
    `absmax_out` (one-element fp32 device tensor) additionally receives max|out|.
    `noalloc` (needs `out`): the entry point that allocates nothing, cn_gemm_f32_noalloc."""
    import torch
    _need(A, torch.float32, "A")
    _need(B, torch.float32, "B")
    M, K = (A.shape[1], A.shape[0]) if trans_a else A.shape
    K2, N = (B.shape[1], B.shape[0]) if trans_b else B.shape
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=A.device)
    _need(out, torch.float32, "out")
    if K != K2 or tuple(out.shape) != (M, N):
        raise CnError(2, "Matrix size error: op(A) %dx%d, op(B) %dx%d, out %dx%d"
                      % (M, K, K2, N, out.shape[0], out.shape[1]))
    if noalloc:
        check(lib().cn_gemm_f32_noalloc(int(trans_a), int(trans_b), M, N, K, A.data_ptr(), _ld(A), B.data_ptr(),
                                        _ld(B), out.data_ptr(), _ld(out), _stream()))
    elif absmax_out is not None:
        _need(absmax_out, torch.float32, "absmax_out")
        check(lib().cn_gemm_f32_absmax(int(trans_a), int(trans_b), M, N, K, A.data_ptr(), _ld(A), B.data_ptr(),
                                       _ld(B), out.data_ptr(), _ld(out), absmax_out.data_ptr(), _stream()))
    else:
        check(lib().cn_gemm_f32(int(trans_a), int(trans_b), M, N, K, A.data_ptr(), _ld(A), B.data_ptr(),
                                _ld(B), out.data_ptr(), _ld(out), _stream()))
    return out


def dot(A, B, out=None, absmax_out=None):
    return gemm(A, B, False, False, out, absmax_out)


def Tdot(A, B, out=None, absmax_out=None):
    return gemm(A, B, True, False, out, absmax_out)


def dotT(A, B, out=None):
    return gemm(A, B, False, True, out)


def gemm_w8(A, W, scale, out=None):
    """out = A decode(W, scale): A fp32 M x K, W uint8 codes K x N."""
    import torch
    _need(A, torch.float32, "A")
    _need(W, torch.uint8, "W")
    M, K = A.shape
    K2, N = W.shape
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=A.device)
    _need(out, torch.float32, "out")
    if K != K2 or tuple(out.shape) != (M, N):
        raise CnError(2, "Matrix size error")
    check(lib().cn_gemm_f32_w8(M, N, K, A.data_ptr(), _ld(A), W.data_ptr(), _ld(W), float(scale),
                               out.data_ptr(), _ld(out), _stream()))
    return out


def gemm_c8c8_add(A, B, precision_a, precision_b, out):
    """out += decodeA(A) decodeB(B): A uint8 codes M x K, B uint8 codes K x N, with kDot8bit's two tables."""
    import torch
    _need(A, torch.uint8, "A")
    _need(B, torch.uint8, "B")
    _need(out, torch.float32, "out")
    M, K = A.shape
    K2, N = B.shape
    if K != K2 or tuple(out.shape) != (M, N):
        raise CnError(2, "Matrix size error")
    check(lib().cn_gemm_c8c8_add(M, N, K, A.data_ptr(), _ld(A), B.data_ptr(), _ld(B), float(precision_a),
                                 float(precision_b), out.data_ptr(), _ld(out), _stream()))
    return out


class Csr:
    """Device CSR matrix: rows x cols, row_ptr (int32, rows + 1), col_idx (int32), vals (fp32)."""

    def __init__(self, rows, cols, row_ptr, col_idx, vals):
        self.rows, self.cols, self.row_ptr, self.col_idx, self.vals = rows, cols, row_ptr, col_idx, vals

    @property
    def nnz(self):
        return self.vals.numel()


def csr_from_dense(A, transpose=False):
    """CSR of the dense row-major A, or of its transpose (the CSC arrays of A)."""
    import torch
    _need(A, torch.float32, "A")
    rows, cols = A.shape
    R, Cc = (cols, rows) if transpose else (rows, cols)
    row_ptr = torch.empty(R + 1, dtype=torch.int32, device=A.device)
    nnz = C.c_int64(0)
    # room for one nonzero in sixteen; a denser matrix reports its count and is converted in a second call
    capacity = max(1024, (rows * cols) // 16)
    while True:
        col_idx = torch.empty(max(capacity, 1), dtype=torch.int32, device=A.device)
        vals = torch.empty(max(capacity, 1), dtype=torch.float32, device=A.device)
        status = lib().cn_csr_from_dense_f32(A.data_ptr(), rows, cols, _ld(A), int(transpose), row_ptr.data_ptr(),
                                             col_idx.data_ptr(), vals.data_ptr(), capacity, C.byref(nnz), _stream())
        if status == 5 and nnz.value > capacity:
            capacity = nnz.value
            continue
        check(status)
        break
    return Csr(R, Cc, row_ptr, col_idx[:nnz.value], vals[:nnz.value])


def csr_gemm(S, B, out=None, absmax_out=None):
    """out = S B (S: Csr of shape R x C, B dense C x N); `absmax_out` (one-element device tensor)
    also receives max|out|."""
    import torch
    _need(B, torch.float32, "B")
    if B.shape[0] != S.cols:
        raise CnError(2, "Matrix size error: S %dx%d, B %dx%d" % (S.rows, S.cols, B.shape[0], B.shape[1]))
    N = B.shape[1]
    if out is None:
        out = torch.empty((S.rows, N), dtype=torch.float32, device=B.device)
    _need(out, torch.float32, "out")
    args = (S.rows, S.cols, N, S.row_ptr.data_ptr(), S.col_idx.data_ptr(), S.vals.data_ptr(), B.data_ptr(), _ld(B),
            out.data_ptr(), _ld(out))
    if absmax_out is None:
        check(lib().cn_csr_gemm_f32(*args, _stream()))
    else:
        _need(absmax_out, torch.float32, "absmax_out")
        check(lib().cn_csr_gemm_f32_absmax(*args, absmax_out.data_ptr(), _stream()))
    return out


def csr_gemm_absmax(S, B, absmax_out=None):
    """max|S B| as a one-element device tensor; the product itself is not stored."""
    import torch
    _need(B, torch.float32, "B")
    if B.shape[0] != S.cols:
        raise CnError(2, "Matrix size error: S %dx%d, B %dx%d" % (S.rows, S.cols, B.shape[0], B.shape[1]))
    if absmax_out is None:
        absmax_out = torch.empty(1, dtype=torch.float32, device=B.device)
    check(lib().cn_csr_gemm_f32_absmax(S.rows, S.cols, B.shape[1], S.row_ptr.data_ptr(), S.col_idx.data_ptr(),
                                       S.vals.data_ptr(), B.data_ptr(), _ld(B), None, 0, absmax_out.data_ptr(), _stream()))
    return absmax_out


def csr_gemm_coded_update(S, B, precision, codes=None, w=None, alpha=1.0):
    """codes of S B at the device scalar `precision`; with `w`, also w += alpha * decode(codes)."""
    import torch
    _need(B, torch.float32, "B")
    _need(precision, torch.float32, "precision")
    if B.shape[0] != S.cols:
        raise CnError(2, "Matrix size error: S %dx%d, B %dx%d" % (S.rows, S.cols, B.shape[0], B.shape[1]))
    N = B.shape[1]
    if codes is None:
        codes = torch.empty((S.rows, N), dtype=torch.uint8, device=B.device)
    _need(codes, torch.uint8, "codes")
    if not codes.is_contiguous() or codes.numel() != S.rows * N:
        raise ValueError("codes must be a contiguous %d x %d uint8 tensor" % (S.rows, N))
    if w is not None:
        _need(w, torch.float32, "w")
        if tuple(w.shape) != (S.rows, N):
            raise CnError(2, "Matrix size error: w %s, S B %dx%d" % (tuple(w.shape), S.rows, N))
    check(lib().cn_csr_gemm_coded_update(S.rows, S.cols, N, S.row_ptr.data_ptr(), S.col_idx.data_ptr(), S.vals.data_ptr(),
                                         B.data_ptr(), _ld(B), precision.data_ptr(), codes.data_ptr(),
                                         None if w is None else w.data_ptr(), 0 if w is None else _ld(w), alpha, _stream()))
    return codes


def csr_gemm_coded_rmsprop(S, B, precision, rms, w, rms_multiplier, learning_rate, codes=None):
    """codes of S B at the device scalar `precision`, then RMSprop with weight update on their decoded values."""
    import torch
    _need(B, torch.float32, "B")
    _need(precision, torch.float32, "precision")
    _need(rms, torch.float32, "rms")
    _need(w, torch.float32, "w")
    N = B.shape[1]
    if B.shape[0] != S.cols or tuple(w.shape) != (S.rows, N) or tuple(rms.shape) != (S.rows, N) or _ld(rms) != _ld(w):
        raise CnError(2, "Matrix size error: S %dx%d, B %s, w %s, rms %s" % (S.rows, S.cols, tuple(B.shape), tuple(w.shape),
                                                                             tuple(rms.shape)))
    if codes is None:
        codes = torch.empty((S.rows, N), dtype=torch.uint8, device=B.device)
    _need(codes, torch.uint8, "codes")
    if not codes.is_contiguous() or codes.numel() != S.rows * N:
        raise ValueError("codes must be a contiguous %d x %d uint8 tensor" % (S.rows, N))
    check(lib().cn_csr_gemm_coded_rmsprop(S.rows, S.cols, N, S.row_ptr.data_ptr(), S.col_idx.data_ptr(), S.vals.data_ptr(),
                                          B.data_ptr(), _ld(B), precision.data_ptr(), codes.data_ptr(), rms.data_ptr(),
                                          w.data_ptr(), _ld(w), rms_multiplier, learning_rate, _stream()))
    return codes


def csr_to_dense(S, out=None):
    import torch
    if out is None:
        out = torch.empty((S.rows, S.cols), dtype=torch.float32, device=S.row_ptr.device)
    _need(out, torch.float32, "out")
    check(lib().cn_csr_to_dense_f32(S.rows, S.cols, S.row_ptr.data_ptr(), S.col_idx.data_ptr(), S.vals.data_ptr(),
                                    out.data_ptr(), _ld(out), _stream()))
    return out


def csr_transpose(S):
    """CSR of S^T."""
    import torch
    dev = S.row_ptr.device
    t_row_ptr = torch.empty(S.cols + 1, dtype=torch.int32, device=dev)
    t_col_idx = torch.empty(max(S.nnz, 1), dtype=torch.int32, device=dev)
    t_vals = torch.empty(max(S.nnz, 1), dtype=torch.float32, device=dev)
    scratch = torch.empty(max(S.cols, 1), dtype=torch.int32, device=dev)
    check(lib().cn_csr_transpose(S.rows, S.cols, S.nnz, S.row_ptr.data_ptr(), S.col_idx.data_ptr(), S.vals.data_ptr(),
                                 t_row_ptr.data_ptr(), t_col_idx.data_ptr(), t_vals.data_ptr(), scratch.data_ptr(),
                                 _stream()))
    return Csr(S.cols, S.rows, t_row_ptr, t_col_idx[:S.nnz], t_vals[:S.nnz])


def absmax(x, out=None):
    """Device scalar max|x| (one-element fp32 tensor)."""
    import torch
    _need(x, torch.float32, "x")
    if not x.is_contiguous():
        raise ValueError("x must be contiguous")
    if out is None:
        out = torch.empty(1, dtype=torch.float32, device=x.device)
    check(lib().cn_absmax_f32(x.data_ptr(), x.numel(), out.data_ptr(), _stream()))
    return out


def compression_8bit(A, precision, out=None):
    """uint8 codes of A / precision; precision is a float or a one-element device tensor."""
    import torch
    _need(A, torch.float32, "A")
    if not A.is_contiguous():
        raise ValueError("A must be contiguous")
    if out is None:
        out = torch.empty(A.shape, dtype=torch.uint8, device=A.device)
    _need(out, torch.uint8, "out")
    if isinstance(precision, torch.Tensor):
        check(lib().cn_compress_8bit_dp(A.data_ptr(), precision.data_ptr(), A.numel(), out.data_ptr(), _stream()))
    else:
        check(lib().cn_compress_8bit(A.data_ptr(), float(precision), A.numel(), out.data_ptr(), _stream()))
    return out


def absmax_compression_8bit(A, out=None, precision_out=None):
    """(codes, precision): precision = max|A| as a one-element device tensor and the codes of A under it, one call."""
    import torch
    _need(A, torch.float32, "A")
    if not A.is_contiguous():
        raise ValueError("A must be contiguous")
    if out is None:
        out = torch.empty(A.shape, dtype=torch.uint8, device=A.device)
    _need(out, torch.uint8, "out")
    if precision_out is None:
        precision_out = torch.empty(1, dtype=torch.float32, device=A.device)
    _need(precision_out, torch.float32, "precision_out")
    check(lib().cn_absmax_compress_8bit(A.data_ptr(), A.numel(), out.data_ptr(), precision_out.data_ptr(), _stream()))
    return out, precision_out


def compression_8bit_axpy(A, precision, alpha, y, out=None):
    """codes of A / precision and y += alpha * decode(codes) in one pass; returns the codes."""
    import torch
    _need(A, torch.float32, "A")
    _need(y, torch.float32, "y")
    if not A.is_contiguous() or not y.is_contiguous() or y.numel() != A.numel():
        raise ValueError("A and y must be contiguous and of one size")
    if out is None:
        out = torch.empty(A.shape, dtype=torch.uint8, device=A.device)
    _need(out, torch.uint8, "out")
    if not out.is_contiguous() or out.numel() != A.numel():
        raise ValueError("out must be a contiguous uint8 tensor of A's size")
    if isinstance(precision, torch.Tensor):
        _need(precision, torch.float32, "precision")
        check(lib().cn_compress_8bit_axpy_dp(A.data_ptr(), precision.data_ptr(), A.numel(), out.data_ptr(), alpha,
                                             y.data_ptr(), _stream()))
    else:
        check(lib().cn_compress_8bit_axpy(A.data_ptr(), float(precision), A.numel(), out.data_ptr(), alpha, y.data_ptr(),
                                          _stream()))
    return out


def decompression_8bit(codes, precision, out=None):
    import torch
    _need(codes, torch.uint8, "codes")
    if not codes.is_contiguous():
        raise ValueError("codes must be contiguous")
    if out is None:
        out = torch.empty(codes.shape, dtype=torch.float32, device=codes.device)
    _need(out, torch.float32, "out")
    if isinstance(precision, torch.Tensor):
        check(lib().cn_decompress_8bit_dp(codes.data_ptr(), precision.data_ptr(), codes.numel(), out.data_ptr(), _stream()))
    else:
        check(lib().cn_decompress_8bit(codes.data_ptr(), float(precision), codes.numel(), out.data_ptr(), _stream()))
    return out


def decode_8bit_lut(codes, lut, out=None):
    """out[i] = lut[codes[i]] for a 256-entry fp32 device table."""
    import torch
    _need(codes, torch.uint8, "codes")
    _need(lut, torch.float32, "lut")
    if not codes.is_contiguous() or lut.numel() != 256 or not lut.is_contiguous():
        raise ValueError("codes must be contiguous and lut a contiguous tensor of 256 floats")
    if out is None:
        out = torch.empty(codes.shape, dtype=torch.float32, device=codes.device)
    _need(out, torch.float32, "out")
    check(lib().cn_decode_8bit_lut(codes.data_ptr(), lut.data_ptr(), codes.numel(), out.data_ptr(), _stream()))
    return out


def decompression_8bit_axpy(codes, precision, alpha, y):
    """y += alpha * decode(codes), in place, one pass."""
    import torch
    _need(codes, torch.uint8, "codes")
    _need(y, torch.float32, "y")
    if not (codes.is_contiguous() and y.is_contiguous()) or codes.numel() != y.numel():
        raise ValueError("codes and y must be contiguous and of equal size")
    if isinstance(precision, torch.Tensor):
        check(lib().cn_decompress_8bit_axpy_dp(codes.data_ptr(), precision.data_ptr(), float(alpha), codes.numel(),
                                               y.data_ptr(), _stream()))
    else:
        check(lib().cn_decompress_8bit_axpy(codes.data_ptr(), float(precision), float(alpha), codes.numel(),
                                            y.data_ptr(), _stream()))
    return y


def rmsprop_update(rms, grad, w, rms_multiplier, learning_rate, precision=None):
    """RMSprop with weight update, in place on rms and w.  `grad` is fp32, or uint8 codes together
    with their `precision` (a float or a one-element device tensor)."""
    import torch
    _need(rms, torch.float32, "rms")
    _need(w, torch.float32, "w")
    if not (rms.is_contiguous() and w.is_contiguous() and grad.is_contiguous()):
        raise ValueError("operands must be contiguous")
    if rms.numel() != w.numel() or grad.numel() != w.numel():
        raise ValueError("operands must be of equal size")
    n = w.numel()
    if grad.dtype == torch.uint8:
        if precision is None:
            raise ValueError("coded gradient needs its precision")
        if isinstance(precision, torch.Tensor):
            check(lib().cn_rmsprop_update_w8_dp(rms.data_ptr(), grad.data_ptr(), precision.data_ptr(), w.data_ptr(),
                                                float(rms_multiplier), float(learning_rate), n, _stream()))
        else:
            check(lib().cn_rmsprop_update_w8(rms.data_ptr(), grad.data_ptr(), float(precision), w.data_ptr(),
                                             float(rms_multiplier), float(learning_rate), n, _stream()))
    else:
        _need(grad, torch.float32, "grad")
        check(lib().cn_rmsprop_update_f32(rms.data_ptr(), grad.data_ptr(), w.data_ptr(), float(rms_multiplier),
                                          float(learning_rate), n, _stream()))
    return rms, w


# ---- small kernels around the path (bias, maxout, softmax, ...) ---------------------------------
def _declare_layers(L):
    i64, vp, f32, sz = C.c_int64, C.c_void_p, C.c_float, C.c_size_t
    L.cn_transpose_f32.argtypes = [vp, i64, i64, vp, vp]
    L.cn_affine_f32.argtypes = [vp, f32, f32, sz, vp, vp]
    L.cn_abs_f32.argtypes = [vp, sz, vp, vp]
    L.cn_sub_f32.argtypes = [vp, vp, sz, vp, vp]
    L.cn_sum_f32.argtypes = [vp, sz, vp, vp]
    L.cn_max_f32.argtypes = [vp, sz, vp, vp]
    L.cn_sgd_update_f32.argtypes = [vp, vp, f32, sz, vp]
    L.cn_add_row_vector_f32.argtypes = [vp, vp, i64, i64, vp, vp]
    L.cn_maxout_f32.argtypes = [vp, i64, i64, C.c_int, vp, vp, vp]
    L.cn_bias_maxout_f32.argtypes = [vp, i64, vp, i64, i64, C.c_int, vp, vp, vp]
    L.cn_gemm_f32_bias_maxout.argtypes = [C.c_int, C.c_int, i64, i64, i64, vp, i64, vp, i64, vp, C.c_int, vp, vp, vp]
    L.cn_gemm_f32_expand_maxout_grad.argtypes = [C.c_int, C.c_int, i64, i64, i64, vp, i64, vp, i64, vp, C.c_int, vp, vp]
    L.cn_csr_gemm_bias_maxout_f32.argtypes = [i64, i64, i64, vp, vp, vp, vp, i64, vp, C.c_int, vp, vp, vp]
    L.cn_expand_to_maxout_grad_f32.argtypes = [vp, vp, i64, i64, C.c_int, vp, vp]
    L.cn_softmax_f32.argtypes = [vp, i64, i64, vp, vp]
    L.cn_timer_start.argtypes = [C.POINTER(vp), vp]
    L.cn_timer_stop.argtypes = [vp, vp, C.POINTER(f32)]
    return L


def _contig(t, what):
    import torch
    _need(t, torch.float32, what)
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % what)
    return t


def transpose(A, out=None):
    import torch
    L = _declare_layers(lib())
    _contig(A, "A")
    if out is None:
        out = torch.empty((A.shape[1], A.shape[0]), dtype=torch.float32, device=A.device)
    check(L.cn_transpose_f32(A.data_ptr(), A.shape[0], A.shape[1], out.data_ptr(), _stream()))
    return out


def add_row_vector(A, v, out=None):
    import torch
    L = _declare_layers(lib())
    _contig(A, "A")
    _contig(v, "v")
    if v.numel() != A.shape[1]:
        raise CnError(2, "vector length %d does not match %d columns" % (v.numel(), A.shape[1]))
    out = torch.empty_like(A) if out is None else out
    check(L.cn_add_row_vector_f32(A.data_ptr(), v.data_ptr(), A.shape[0], A.shape[1], out.data_ptr(), _stream()))
    return out


def maxout(A, pool):
    import torch
    L = _declare_layers(lib())
    _contig(A, "A")
    out = torch.empty((A.shape[0], A.shape[1] // pool), dtype=torch.float32, device=A.device)
    arg = torch.empty_like(out)
    check(L.cn_maxout_f32(A.data_ptr(), A.shape[0], A.shape[1], int(pool), out.data_ptr(), arg.data_ptr(), _stream()))
    return out, arg


def bias_maxout(A, v, pool):
    """maxout(A + v) with v added to every row: (values, winners' columns), the sum never stored."""
    import torch
    L = _declare_layers(lib())
    _need(A, torch.float32, "A")
    _contig(v, "v")
    if v.numel() != A.shape[1] or A.shape[1] % pool:
        raise CnError(2, "Matrix size error: A %s, v %d, pool %d" % (tuple(A.shape), v.numel(), pool))
    out = torch.empty((A.shape[0], A.shape[1] // pool), dtype=torch.float32, device=A.device)
    arg = torch.empty_like(out)
    check(L.cn_bias_maxout_f32(A.data_ptr(), _ld(A), v.data_ptr(), A.shape[0], A.shape[1], int(pool), out.data_ptr(),
                               arg.data_ptr(), _stream()))
    return out, arg


def dot_bias_maxout(A, B, v, pool):
    """maxout(A B + v): (values, winners' columns); bias and maxout ride on the product's chunk sum."""
    import torch
    L = _declare_layers(lib())
    _need(A, torch.float32, "A")
    _need(B, torch.float32, "B")
    _contig(v, "v")
    M, K = A.shape
    K2, N = B.shape
    if K != K2 or v.numel() != N or N % pool:
        raise CnError(2, "Matrix size error: A %s, B %s, v %d, pool %d" % (tuple(A.shape), tuple(B.shape), v.numel(), pool))
    out = torch.empty((M, N // pool), dtype=torch.float32, device=A.device)
    arg = torch.empty_like(out)
    check(L.cn_gemm_f32_bias_maxout(0, 0, M, N, K, A.data_ptr(), _ld(A), B.data_ptr(), _ld(B), v.data_ptr(), int(pool),
                                    out.data_ptr(), arg.data_ptr(), _stream()))
    return out, arg


def dotT_expand_to_maxout_grad(E, W, argmax, pool):
    """expand_to_maxout_grad(E W^T, argmax): the error of the layer below, in the winners' columns."""
    import torch
    L = _declare_layers(lib())
    _need(E, torch.float32, "E")
    _need(W, torch.float32, "W")
    _contig(argmax, "argmax")
    M, K = E.shape
    N, K2 = W.shape
    if K != K2 or tuple(argmax.shape) != (M, N):
        raise CnError(2, "Matrix size error: E %s, W %s, argmax %s" % (tuple(E.shape), tuple(W.shape), tuple(argmax.shape)))
    out = torch.empty((M, N * pool), dtype=torch.float32, device=E.device)
    check(L.cn_gemm_f32_expand_maxout_grad(0, 1, M, N, K, E.data_ptr(), _ld(E), W.data_ptr(), _ld(W), argmax.data_ptr(),
                                           int(pool), out.data_ptr(), _stream()))
    return out


def csr_gemm_bias_maxout(S, B, v, pool):
    """maxout(S B + v): (values, winners' columns) of the first layer on a sparse batch."""
    import torch
    L = _declare_layers(lib())
    _need(B, torch.float32, "B")
    _contig(v, "v")
    N = B.shape[1]
    if B.shape[0] != S.cols or v.numel() != N or N % pool:
        raise CnError(2, "Matrix size error: S %dx%d, B %s, v %d, pool %d" % (S.rows, S.cols, tuple(B.shape), v.numel(), pool))
    out = torch.empty((S.rows, N // pool), dtype=torch.float32, device=B.device)
    arg = torch.empty_like(out)
    check(L.cn_csr_gemm_bias_maxout_f32(S.rows, S.cols, N, S.row_ptr.data_ptr(), S.col_idx.data_ptr(), S.vals.data_ptr(),
                                        B.data_ptr(), _ld(B), v.data_ptr(), int(pool), out.data_ptr(), arg.data_ptr(), _stream()))
    return out, arg


def expand_to_maxout_grad(err, argmax, pool, out=None):
    import torch
    L = _declare_layers(lib())
    _contig(err, "err")
    _contig(argmax, "argmax")
    if out is None:
        out = torch.empty((err.shape[0], err.shape[1] * pool), dtype=torch.float32, device=err.device)
    check(L.cn_expand_to_maxout_grad_f32(err.data_ptr(), argmax.data_ptr(), err.shape[0], err.shape[1], int(pool),
                                         out.data_ptr(), _stream()))
    return out


def softmax(A, out=None):
    import torch
    L = _declare_layers(lib())
    _contig(A, "A")
    out = torch.empty_like(A) if out is None else out
    check(L.cn_softmax_f32(A.data_ptr(), A.shape[0], A.shape[1], out.data_ptr(), _stream()))
    return out


def fill(t, value):
    """t[:] = value on a contiguous fp32 device tensor (the reference's zeros / ones / fill)."""
    import torch
    _need(t, torch.float32, "t")
    if not t.is_contiguous():
        raise ValueError("t must be contiguous")
    check(lib().cn_fill_f32(t.data_ptr(), float(value), t.numel(), _stream()))
    return t


def sub(a, b, out=None):
    import torch
    L = _declare_layers(lib())
    _contig(a, "a")
    _contig(b, "b")
    out = torch.empty_like(a) if out is None else out
    check(L.cn_sub_f32(a.data_ptr(), b.data_ptr(), a.numel(), out.data_ptr(), _stream()))
    return out


def sgd_update(w, grad, rate):
    L = _declare_layers(lib())
    _contig(w, "w")
    _contig(grad, "grad")
    check(L.cn_sgd_update_f32(w.data_ptr(), grad.data_ptr(), float(rate), w.numel(), _stream()))
    return w


def reduce_sum(x):
    import torch
    L = _declare_layers(lib())
    _contig(x, "x")
    out = torch.empty(1, dtype=torch.float32, device=x.device)
    check(L.cn_sum_f32(x.data_ptr(), x.numel(), out.data_ptr(), _stream()))
    return out


def reduce_max(x):
    import torch
    L = _declare_layers(lib())
    _contig(x, "x")
    out = torch.empty(1, dtype=torch.float32, device=x.device)
    check(L.cn_max_f32(x.data_ptr(), x.numel(), out.data_ptr(), _stream()))
    return out

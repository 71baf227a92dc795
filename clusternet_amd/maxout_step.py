"""One training step of a maxout MLP written against the path's operators, the way the reference's
callers compose them (forward: source/test.cu:266-291 and source/Layer.cpp:250-261; backward:
source/Layer.cpp:314-339; 8-bit gradient round trip: source/Layer.cpp:365,433 and
source/DeepNeuralNetwork.cpp:334-339).  Host-side glue only: every array operation is one call
into libcnhip.

    z1 = X W1 + b1;  h1, a1 = maxout(z1);  z2 = h1 W2 + b2;  h2, a2 = maxout(z2)
    p  = softmax(h2 W3 + b3);  e3 = p - onehot(y)
    gW3 = h2^T e3;  e2 = expand(e3 W3^T, a2);  gW2 = h1^T e2;  e1 = expand(e2 W2^T, a1);  gW1 = X^T e1
    each gW -> absmax -> compression_8bit -> W -= rate * decode(codes)   (one fused pass, identical
    bit for bit to decompression_8bit followed by the update)
Biases are inputs and are not updated.

A sparse batch (the reference feeds its 2 % dense inputs as sparse matrices, source/Layer.cpp:250-255
and 318-321) goes in as `sparse_input(X)`: the first layer's product and its weight gradient then run
on the compressed rows of X and of X^T.
"""
from . import _lib as L


class SparseInput:
    """X in compressed sparse rows together with X^T in the same form."""

    def __init__(self, csr, csr_t):
        self.csr, self.csr_t = csr, csr_t


def sparse_input(X):
    csr = L.csr_from_dense(X)
    return SparseInput(csr, L.csr_transpose(csr))


def forward(X, params, pool=2):
    W1, b1, W2, b2, W3, b3 = params
    # bias and maxout are taken in one pass behind each product (inside it for the sparse first layer)
    if isinstance(X, SparseInput):
        h1, a1 = L.csr_gemm_bias_maxout(X.csr, W1, b1, pool)
    else:
        h1, a1 = L.dot_bias_maxout(X, W1, b1, pool)
    h2, a2 = L.dot_bias_maxout(h1, W2, b2, pool)
    p = L.softmax(L.add_row_vector(L.dot(h2, W3), b3))
    return p, (h1, a1, h2, a2)


def backward(X, onehot, params, p, cache, pool=2, absmax_out=None, defer_first=False):
    """Weight gradients.  `absmax_out` = three one-element device tensors: the gradient products then
    also deliver max|gW|, which saves the abs-max pass in front of compression_8bit.
    `defer_first` (sparse input only): the first element of the result is the error signal e1 instead
    of gW1 = X^T e1, for `coded_sparse_update`, which never stores that gradient."""
    W1, b1, W2, b2, W3, b3 = params
    h1, a1, h2, a2 = cache
    m1, m2, m3 = absmax_out if absmax_out is not None else (None, None, None)
    e3 = L.sub(p, onehot)
    gW3 = L.Tdot(h2, e3, absmax_out=m3)
    e2 = L.dotT_expand_to_maxout_grad(e3, W3, a2, pool)
    gW2 = L.Tdot(h1, e2, absmax_out=m2)
    e1 = L.dotT_expand_to_maxout_grad(e2, W2, a1, pool)
    if isinstance(X, SparseInput) and defer_first:
        gW1 = e1
    elif isinstance(X, SparseInput):
        gW1 = L.csr_gemm(X.csr_t, e1, absmax_out=m1)
    else:
        gW1 = L.Tdot(X, e1, absmax_out=m1)
    return gW1, gW2, gW3


def codec_round_trip(grad):
    """absmax -> compression_8bit -> decompression_8bit without a host synchronisation."""
    prec = L.absmax(grad)
    codes = L.compression_8bit(grad, prec)
    return L.decompression_8bit(codes, prec, out=grad), codes, prec


def coded_update(w, grad, rate, fused=True, scratch=None, prec=None):
    """W -= rate * decode(encode(grad)).  `fused` picks the one-pass kernel; the unfused sequence
    (decompression_8bit into `scratch`, or over `grad` itself, then the update) gives the same bits.
    `prec` = max|grad| on the device if the caller already has it."""
    if prec is None:
        prec = L.absmax(grad)
    if fused:
        return L.compression_8bit_axpy(grad, prec, -rate, w), prec
    codes = L.compression_8bit(grad, prec)
    L.sgd_update(w, L.decompression_8bit(codes, prec, out=grad if scratch is None else scratch), rate)
    return codes, prec


def coded_sparse_update(w, Xs, e1, rate, prec=None, codes=None):
    """W -= rate * decode(encode(X^T e1)) for a sparse batch without the gradient ever reaching memory:
    one pass for max|X^T e1|, one that recomputes each gradient row from its two or three nonzeros,
    encodes it (the codes are what the exchange between GPUs sends) and updates the weights.  Bit for bit
    the result of csr_gemm, absmax, compression_8bit and decompression_8bit_axpy."""
    prec = L.csr_gemm_absmax(Xs.csr_t, e1, prec)
    codes = L.csr_gemm_coded_update(Xs.csr_t, e1, prec, codes, w=w, alpha=-rate)
    return codes, prec


def coded_sparse_rmsprop_update(w, rms, Xs, e1, rms_multiplier, rate, prec=None, codes=None):
    """RMSprop with weight update on the 8-bit round trip of X^T e1 for a sparse batch, the gradient never
    stored: the RMSprop form of `coded_sparse_update`."""
    prec = L.csr_gemm_absmax(Xs.csr_t, e1, prec)
    codes = L.csr_gemm_coded_rmsprop(Xs.csr_t, e1, prec, rms, w, rms_multiplier, rate, codes)
    return codes, prec


def coded_rmsprop_update(w, rms, grad, rms_multiplier, rate, fused=True, scratch=None):
    """RMSprop with weight update (source/basicOps.cu:1192-1197) on the 8-bit round trip of `grad`."""
    prec = L.absmax(grad)
    codes = L.compression_8bit(grad, prec)
    if fused:
        L.rmsprop_update(rms, codes, w, rms_multiplier, rate, precision=prec)
    else:
        L.rmsprop_update(rms, L.decompression_8bit(codes, prec, out=grad if scratch is None else scratch), w,
                         rms_multiplier, rate)
    return codes, prec


def step(X, onehot, params, rate, pool=2):
    import torch
    p, cache = forward(X, params, pool)
    maxima = [torch.empty(1, dtype=torch.float32, device=p.device) for _ in range(3)]
    sparse = isinstance(X, SparseInput)
    grads = backward(X, onehot, params, p, cache, pool, absmax_out=maxima, defer_first=sparse)
    W = (params[0], params[2], params[4])
    for i, (w, g, m) in enumerate(zip(W, grads, maxima)):
        if sparse and i == 0:
            coded_sparse_update(w, X, g, rate, prec=m)
        else:
            coded_update(w, g, rate, prec=m)
    return p

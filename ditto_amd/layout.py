"""The reference's packed conv placeholders <-> the plain NCHW / KCRS tensors the kernels take.

The reference's GPU conv drivers hand over tensors the host has packed in blocks of 16 channels and padded
(benchmark/chimera/cuda/conv3x3_conv1x1_cuda.py:90-105, 164-170):

    Img[N, C/16, H + 2 pad, W + 2 pad (+ slack), 16]     already padded: the border is part of the tensor
    W1 [R, S, C/16, K1/16, 16, 16]                        (r, s, c outer, k1 outer, c inner, k1 inner)
    W2 [K1/16, K2/16, 16, 16]       (1x1 second filter)   (k1 outer, k2 outer, k1 inner, k2 inner)
    W2 [R2, S2, K1/16, K2/16, 16, 16]                     (a larger second filter, conv1x1_conv3x3_cuda.py:95-99)
    Out[N, K2/16, P, Q, 16]

The kernels of this package read NCHW.  These functions convert on the device with torch's own copy kernels, one
pass per tensor: a caller that holds packed tensors gets the reference's calling convention at the price of those
passes (an image and an output pass per call; the weights once, when the function is specialised).  A first
convolution on a packed image runs with padding 0 over the padded tensor, so whatever the caller put into the
border takes part exactly as in the reference's index expression.  Stride 1 only: the reference's padded width
depends on its strides in a way its own index expression does not use (``Q + stride1 + 2`` columns, of which
``Q + 2`` are read, :100 and :112).
"""
import torch

BLOCK = 16


def unpack_image(img_p, cols=None):
    """Img[N, C/16, Hp, Wp, 16] -> X[N, C, Hp, cols] (contiguous); ``cols``: the columns that are read (default all)."""
    n, co, hp, wp, ci = img_p.shape
    if ci != BLOCK:
        raise ValueError("packed image must end in a block of %d channels" % BLOCK)
    x = img_p if cols is None else img_p[:, :, :, :cols, :]
    return x.permute(0, 1, 4, 2, 3).reshape(n, co * BLOCK, hp, x.shape[3]).contiguous()


def pack_image(x, pad=0, slack=0):
    """X[N, C, H, W] -> Img[N, C/16, H + 2 pad, W + 2 pad + slack, 16] with a zero border."""
    n, c, h, w = x.shape
    if c % BLOCK:
        raise ValueError("channels must be a multiple of %d" % BLOCK)
    out = torch.zeros(n, c // BLOCK, h + 2 * pad, w + 2 * pad + slack, BLOCK, dtype=x.dtype, device=x.device)
    out[:, :, pad:pad + h, pad:pad + w, :] = x.reshape(n, c // BLOCK, BLOCK, h, w).permute(0, 1, 3, 4, 2)
    return out


def unpack_weight(w_p):
    """W[R, S, C/16, K/16, 16, 16] (or the 1x1 form [C/16, K/16, 16, 16]) -> W[K, C, R, S]."""
    if w_p.dim() == 4:
        w_p = w_p[None, None]
    r, s, co, ko, ci, ki = w_p.shape
    if ci != BLOCK or ki != BLOCK:
        raise ValueError("packed weights must end in 16 x 16 blocks")
    return w_p.permute(3, 5, 2, 4, 0, 1).reshape(ko * BLOCK, co * BLOCK, r, s).contiguous()


def pack_weight(w, one_by_one_as_4d=True):
    """W[K, C, R, S] -> the packed form above."""
    k, c, r, s = w.shape
    if k % BLOCK or c % BLOCK:
        raise ValueError("channels must be multiples of %d" % BLOCK)
    p = w.reshape(k // BLOCK, BLOCK, c // BLOCK, BLOCK, r, s).permute(4, 5, 2, 0, 3, 1).contiguous()
    return p[0, 0] if (r == 1 and s == 1 and one_by_one_as_4d) else p


def pack_output_into(y, out_p):
    """Y[N, K, P, Q] -> Out[N, K/16, P, Q', 16] in place (Q' >= Q: the reference rounds Q up to 16; columns beyond Q
    are left as they are)."""
    n, k, p, q = y.shape
    if tuple(out_p.shape[:3]) != (n, k // BLOCK, p) or out_p.shape[3] < q or out_p.shape[4] != BLOCK:
        raise ValueError("packed output must be [%d, %d, %d, >= %d, %d], got %s" % (n, k // BLOCK, p, q, BLOCK,
                                                                                   tuple(out_p.shape)))
    out_p[:, :, :, :q, :] = y.reshape(n, k // BLOCK, BLOCK, p, q).permute(0, 1, 3, 4, 2)
    return out_p

"""Packed (channel-blocked) tensor layout of the SMaLL layer API, channel block 16.

Mirrors include/small/buffers.hpp:33-120, 138-283 of the reference (pack_buffer / unpack_buffer and
the index maps) as vectorised numpy reshapes:
  activations  NCHW  -> [N][C/cb][H][W][cb]        (cb = C when C in {1,2,3})
  conv filter  OIHW  -> [Co/16][Ci/cib][kh][kw][cib][16]
  dw filter    C1HW  -> [C/16][kh][kw][16]
"""
import numpy as np

CB = 16


def in_block(channels, cb=CB):
    if channels % cb == 0:
        return cb
    if channels in (1, 2, 3) and channels < cb:
        return channels
    raise ValueError("channel count %d is neither a multiple of %d nor 1, 2 or 3" % (channels, cb))


def pad_channels(c, cb=CB):
    return (c + cb - 1) // cb * cb


def pack_activations(x, cb=CB):
    """x: [N, C, H, W] -> flat packed array."""
    x = np.asarray(x)
    n, c, h, w = x.shape
    b = in_block(c, cb)
    return np.ascontiguousarray(x.reshape(n, c // b, b, h, w).transpose(0, 1, 3, 4, 2)).ravel()


def unpack_activations(p, n, c, h, w, cb=CB):
    b = in_block(c, cb)
    return np.ascontiguousarray(np.asarray(p).reshape(n, c // b, h, w, b).transpose(0, 1, 4, 2, 3)).reshape(n, c, h, w)


def pack_conv_filter(f, cb=CB, pad_output=True):
    """f: [Co, Ci, kh, kw]; Co is zero-padded up to a multiple of cb
    (what Conv2DLayer does, include/small/Conv2DLayer.hpp:393-404)."""
    f = np.asarray(f)
    co, ci, kh, kw = f.shape
    cop = pad_channels(co, cb) if pad_output else co
    if cop != co:
        f = np.concatenate([f, np.zeros((cop - co, ci, kh, kw), f.dtype)], 0)
    ib = in_block(ci, cb)
    return np.ascontiguousarray(
        f.reshape(cop // cb, cb, ci // ib, ib, kh, kw).transpose(0, 2, 4, 5, 3, 1)).ravel()


def pack_dw_filter(f, cb=CB):
    """f: [C, 1, kh, kw] or [C, kh, kw]."""
    f = np.asarray(f)
    if f.ndim == 4:
        f = f[:, 0]
    c, kh, kw = f.shape
    return np.ascontiguousarray(f.reshape(c // cb, cb, kh, kw).transpose(0, 2, 3, 1)).ravel()


def pack_dense_filter(f, cb=CB):
    """f: [No, Ni] -> the 1x1 convolution filter layout."""
    f = np.asarray(f)
    return pack_conv_filter(f.reshape(f.shape[0], f.shape[1], 1, 1), cb)


def pack_bias(b, cb=CB):
    b = np.asarray(b)
    cop = pad_channels(b.size, cb)
    return np.concatenate([b, np.zeros(cop - b.size, b.dtype)]) if cop != b.size else b.copy()

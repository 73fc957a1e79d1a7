"""Independent restatements used to pin the oracle (and nothing else).

They are written from the mathematical definition, not from the oracle's code: explicit zero
padding + window slicing for convolutions, exact rationals for rounding.
"""
from fractions import Fraction
import math

import numpy as np


def round_half_up_exact(v, shift):
    """floor(v / 2^shift + 1/2) in exact rationals; shift <= 0 is a plain multiplication."""
    if shift <= 0:
        return v * (1 << -shift)
    return math.floor(Fraction(v, 1 << shift) + Fraction(1, 2))


def round_half_even_exact(v, shift):
    if shift <= 0:
        return v * (1 << -shift)
    return round(Fraction(v, 1 << shift))  # Python rounds exact ties to even


def requant_vec(acc, shift, relu, lo, hi, half_even=False):
    """acc: int64 array [..., OC]; shift: array broadcastable on the last axis."""
    acc = np.asarray(acc, dtype=np.int64)
    shift = np.broadcast_to(np.asarray(shift, dtype=np.int64), acc.shape)
    out = np.empty(acc.shape, dtype=np.int64)
    fn = round_half_even_exact if half_even else round_half_up_exact
    flat_a, flat_s, flat_o = acc.ravel(), shift.ravel(), out.ravel()
    if half_even or flat_a.size < 4096:
        for i in range(flat_a.size):
            flat_o[i] = max(min(fn(int(flat_a[i]), int(flat_s[i])), 2**40), -2**40)
    else:
        # float64 is exact here: |acc| < 2^45 and 2^shift is a power of two
        pos = flat_s > 0
        scaled = np.where(pos, flat_a / np.exp2(np.where(pos, flat_s, 0)) + 0.5, 0.0)
        flat_o[:] = np.where(pos, np.floor(scaled).astype(np.int64),
                             flat_a * (np.int64(1) << np.where(pos, 0, -flat_s)))
    if relu:
        out = np.maximum(out, 0)
    return np.clip(out, lo, hi)


def pad_nhwc(x, pads):
    t, b, l, r = pads
    return np.pad(x, ((0, 0), (t, b), (l, r), (0, 0)))


def conv2d_acc(x, w_ockkc, stride, dilation, pads):
    """Dense conv accumulators (int64). x [N,H,W,C]; w [OC,KH,KW,C]."""
    x = pad_nhwc(np.asarray(x, dtype=np.int64), pads)
    w = np.asarray(w_ockkc, dtype=np.int64)
    oc, kh, kw, c = w.shape
    n, hp, wp, _ = x.shape
    oh = (hp - dilation[0] * (kh - 1) - 1) // stride[0] + 1
    ow = (wp - dilation[1] * (kw - 1) - 1) // stride[1] + 1
    acc = np.zeros((n, oh, ow, oc), dtype=np.int64)
    for ky in range(kh):
        for kx in range(kw):
            y0, x0 = ky * dilation[0], kx * dilation[1]
            patch = x[:, y0:y0 + (oh - 1) * stride[0] + 1:stride[0], x0:x0 + (ow - 1) * stride[1] + 1:stride[1], :]
            acc += np.tensordot(patch, w[:, ky, kx, :], axes=([3], [1]))
    return acc


def depthwise_acc(x, w_kkc, stride, dilation, pads):
    x = pad_nhwc(np.asarray(x, dtype=np.int64), pads)
    w = np.asarray(w_kkc, dtype=np.int64)
    kh, kw, c = w.shape
    n, hp, wp, _ = x.shape
    oh = (hp - dilation[0] * (kh - 1) - 1) // stride[0] + 1
    ow = (wp - dilation[1] * (kw - 1) - 1) // stride[1] + 1
    acc = np.zeros((n, oh, ow, c), dtype=np.int64)
    for ky in range(kh):
        for kx in range(kw):
            y0, x0 = ky * dilation[0], kx * dilation[1]
            patch = x[:, y0:y0 + (oh - 1) * stride[0] + 1:stride[0], x0:x0 + (ow - 1) * stride[1] + 1:stride[1], :]
            acc += patch * w[ky, kx, :]
    return acc


def conv2d_ref(x, w, bias, shift, stride, dilation, pads, relu, bits=8, half_even=False):
    acc = conv2d_acc(x, w, stride, dilation, pads)
    if bias is not None:
        acc = acc + np.asarray(bias, dtype=np.int64)
    lo, hi = (-128, 127) if bits == 8 else (-32768, 32767)
    dt = np.int8 if bits == 8 else np.int16
    return requant_vec(acc, shift, relu, lo, hi, half_even).astype(dt)


def depthwise_ref(x, w, bias, shift, stride, dilation, pads, relu, bits=8, half_even=False):
    acc = depthwise_acc(x, w, stride, dilation, pads)
    if bias is not None:
        acc = acc + np.asarray(bias, dtype=np.int64)
    lo, hi = (-128, 127) if bits == 8 else (-32768, 32767)
    dt = np.int8 if bits == 8 else np.int16
    return requant_vec(acc, shift, relu, lo, hi, half_even).astype(dt)

"""Seeded synthetic inputs for the parity tests (numpy only; no reference code involved)."""
import numpy as np


def ternary_matrix(rng, rows, cols, p_zero=0.42):
    """i.i.d. entries: P(0)=p_zero, P(+1)=P(-1)=(1-p_zero)/2, int8 [rows, cols]."""
    u = rng.random((rows, cols))
    w = np.zeros((rows, cols), np.int8)
    half = (1.0 - p_zero) / 2.0
    w[u < half] = 1
    w[(u >= half) & (u < 2 * half)] = -1
    return w


def pack_np(w):
    """Independent packer: numpy packbits, LSB-first, 32 columns per uint32 word."""
    rows, cols = w.shape
    assert cols % 32 == 0
    nz = np.packbits((w != 0).astype(np.uint8), axis=1, bitorder="little")
    sg = np.packbits((w > 0).astype(np.uint8), axis=1, bitorder="little")
    return (np.ascontiguousarray(nz).view("<u4").reshape(rows, cols // 32),
            np.ascontiguousarray(sg).view("<u4").reshape(rows, cols // 32))


def unpack_np(nz, sg):
    """Independent unpacker via numpy unpackbits; sign bits under clear nz bits are ignored."""
    rows, words = nz.shape
    nzb = np.unpackbits(np.ascontiguousarray(nz).view(np.uint8), axis=1, bitorder="little")
    sgb = np.unpackbits(np.ascontiguousarray(sg).view(np.uint8), axis=1, bitorder="little")
    return (nzb.astype(np.int8) * (2 * sgb.astype(np.int8) - 1)).reshape(rows, words * 32)


def scales_f16(rng, rows, groups, lo=0.01, hi=0.03):
    return rng.uniform(lo, hi, (rows, groups)).astype(np.float16)


def acts_f16(rng, *shape, unit_rms=False):
    x = rng.standard_normal(shape)
    if unit_rms:
        x = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True))
    return x.astype(np.float16)


def dense_f64(nz, sg, scales, group=128):
    """Dense float64 matrix W*S with every weight multiplied by its group's scale."""
    w = unpack_np(nz, sg).astype(np.float64)
    s = np.repeat(np.asarray(scales, np.float16).astype(np.float64), group, axis=1)
    return w * s[:, : w.shape[1]]


def problem(seed, rows, cols, p_zero=0.42, group=128, dontcare_sign=False, lo=0.01, hi=0.03,
            unit_rms=False):
    rng = np.random.default_rng(seed)
    w = ternary_matrix(rng, rows, cols, p_zero)
    nz, sg = pack_np(w)
    if dontcare_sign:  # random sign bits under zero weights: must not change any result
        sg = sg | (rng.integers(0, 2**32, nz.shape, dtype=np.uint64).astype(np.uint32) & ~nz)
    s = scales_f16(rng, rows, cols // group, lo, hi)
    x = acts_f16(rng, cols, unit_rms=unit_rms)
    return nz, sg, s, x

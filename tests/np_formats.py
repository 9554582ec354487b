"""Independent, vectorised NumPy restatement of the block formats (test-side cross-check of the C oracle).

Written from the published layouts with array indexing instead of the oracle's
scalar loops, so that an indexing slip in either shows up as a mismatch.
"""
import numpy as np


def f16(bytes2: np.ndarray) -> np.ndarray:
    """little-endian byte pairs [..., 2] -> float32"""
    return np.ascontiguousarray(bytes2).view(np.float16)[..., 0].astype(np.float32)


def dequant_q4_0(packed: np.ndarray, k: int) -> np.ndarray:
    n = packed.shape[0]
    b = packed.reshape(n, k // 32, 18)
    d = f16(b[:, :, 0:2])
    qs = b[:, :, 2:].astype(np.int32)
    q = np.concatenate([qs & 15, qs >> 4], axis=2) - 8  # elements 0..15 low nibbles, 16..31 high
    return (q.astype(np.float32) * d[:, :, None]).reshape(n, k)


def unpack_scales_q4_k(s: np.ndarray):
    """s [..., 12] uint8 -> (sc [..., 8], mn [..., 8])"""
    s = s.astype(np.int32)
    sc = np.empty(s.shape[:-1] + (8,), np.int32)
    mn = np.empty_like(sc)
    sc[..., :4] = s[..., 0:4] & 63
    mn[..., :4] = s[..., 4:8] & 63
    sc[..., 4:] = (s[..., 8:12] & 15) | ((s[..., 0:4] >> 6) << 4)
    mn[..., 4:] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
    return sc, mn


def dequant_q4_k(packed: np.ndarray, k: int) -> np.ndarray:
    n = packed.shape[0]
    b = packed.reshape(n, k // 256, 144)
    d, dmin = f16(b[:, :, 0:2]), f16(b[:, :, 2:4])
    sc, mn = unpack_scales_q4_k(b[:, :, 4:16])
    qs = b[:, :, 16:].reshape(n, k // 256, 4, 32).astype(np.int32)
    q = np.stack([qs & 15, qs >> 4], axis=3).reshape(n, k // 256, 8, 32)  # sub-block 2c low, 2c+1 high
    dl = (d[:, :, None] * sc.astype(np.float32)).astype(np.float32)
    ml = (dmin[:, :, None] * mn.astype(np.float32)).astype(np.float32)
    w = (dl[..., None] * q.astype(np.float32)).astype(np.float32) - ml[..., None]
    return w.astype(np.float32).reshape(n, k)


def dequant_q5_k(packed: np.ndarray, k: int) -> np.ndarray:
    """176-byte blocks: f16 d, f16 dmin, 12 B scales (as Q4_K), qh[32], qs[128]; the fifth bit of sub-block j's
    codes is bit j of the qh byte at the code's position in the sub-block."""
    n = packed.shape[0]
    b = packed.reshape(n, k // 256, 176)
    d, dmin = f16(b[:, :, 0:2]), f16(b[:, :, 2:4])
    sc, mn = unpack_scales_q4_k(b[:, :, 4:16])
    qh = b[:, :, 16:48].astype(np.int32)                                   # [n, nb, 32]
    qs = b[:, :, 48:].reshape(n, k // 256, 4, 32).astype(np.int32)
    low = np.stack([qs & 15, qs >> 4], axis=3).reshape(n, k // 256, 8, 32)  # sub-block 2c low nibbles, 2c+1 high
    fifth = (qh[:, :, None, :] >> np.arange(8)[None, None, :, None]) & 1    # [n, nb, 8, 32]
    q = low + 16 * fifth
    dl = (d[:, :, None] * sc.astype(np.float32)).astype(np.float32)
    ml = (dmin[:, :, None] * mn.astype(np.float32)).astype(np.float32)
    w = (dl[..., None] * q.astype(np.float32)).astype(np.float32) - ml[..., None]
    return w.astype(np.float32).reshape(n, k)


def dequant_q6_k(packed: np.ndarray, k: int) -> np.ndarray:
    n = packed.shape[0]
    b = packed.reshape(n, k // 256, 210)
    ql = b[:, :, 0:128].reshape(n, -1, 2, 64).astype(np.int32)
    qh = b[:, :, 128:192].reshape(n, -1, 2, 32).astype(np.int32)
    sc = b[:, :, 192:208].view(np.int8).reshape(n, -1, 2, 8).astype(np.float32)
    d = f16(b[:, :, 208:210])
    lo = np.stack([ql[..., :32] & 15, ql[..., 32:] & 15, ql[..., :32] >> 4, ql[..., 32:] >> 4], axis=3)  # [n,b,2,4,32]
    hi = np.stack([(qh >> s) & 3 for s in (0, 2, 4, 6)], axis=3)
    q = (lo | (hi << 4)) - 32
    # scale index inside a half: 2*quarter + (l // 16)
    idx = (2 * np.arange(4)[:, None] + (np.arange(32) // 16)[None, :])
    scq = np.take_along_axis(sc[:, :, :, None, :].repeat(4, axis=3), idx[None, None, None].repeat(n, 0).repeat(sc.shape[1], 1).repeat(2, 2), axis=4)
    w = (d[:, :, None, None, None] * scq).astype(np.float32) * q.astype(np.float32)
    return w.astype(np.float32).reshape(n, k)


def dequant_gptq(qweight, scales_u16, qzeros, group=128, g_idx=None) -> np.ndarray:
    """-> [N, K] float32"""
    k8, n = qweight.shape
    k = k8 * 8
    shifts = (4 * np.arange(8, dtype=np.uint32))
    q = ((qweight.view(np.uint32)[:, None, :] >> shifts[None, :, None]) & 15).reshape(k, n).astype(np.int32)
    z = ((qzeros.view(np.uint32)[:, :, None] >> shifts[None, None, :]) & 15).reshape(qzeros.shape[0], n).astype(np.int32) + 1
    s = scales_u16.view(np.float16).astype(np.float32)
    g = np.arange(k) // group if g_idx is None else np.asarray(g_idx, np.int64)
    w = s[g, :] * (q - z[g, :]).astype(np.float32)
    return np.ascontiguousarray(w.T.astype(np.float32))


def gptq_act_order(qweight_sorted, perm, group=128):
    """An act-order (desc_act=True) checkpoint from tensors quantised in sorted order.

    `qweight_sorted` packs the weight whose input columns were taken in the order `perm` (sorted position p
    holds original column perm[p]), quantised with plain groups of `group` sorted positions.  AutoGPTQ stores
    such a layer with the rows of qweight back in the original order and `g_idx[perm[p]] = p // group`;
    scales and qzeros stay as they are.  Returns (qweight int32[K/8, N], g_idx int32[K]).
    """
    k8, n = qweight_sorted.shape
    k = k8 * 8
    perm = np.asarray(perm, np.int64)
    assert sorted(perm.tolist()) == list(range(k))
    shifts = 4 * np.arange(8, dtype=np.uint32)
    nib = ((qweight_sorted.view(np.uint32)[:, None, :] >> shifts[None, :, None]) & 15).reshape(k, n)
    orig = np.empty_like(nib)
    orig[perm] = nib
    packed = (orig.reshape(k8, 8, n).astype(np.uint32) << shifts[None, :, None]).sum(axis=1, dtype=np.uint64).astype(np.uint32)
    g_idx = np.empty(k, np.int32)
    g_idx[perm] = (np.arange(k) // group).astype(np.int32)
    return np.ascontiguousarray(packed).view(np.int32), g_idx


def quantize_q4_0(x: np.ndarray) -> np.ndarray:
    n, k = x.shape
    xb = x.reshape(n, k // 32, 32)
    idx = np.argmax(np.abs(xb), axis=2)  # first maximum
    mx = np.take_along_axis(xb, idx[..., None], axis=2)[..., 0]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
    t = (xb * inv[..., None]).astype(np.float32) + np.float32(8.5)
    q = np.minimum(t.astype(np.int32), 15).astype(np.uint8)
    out = np.empty((n, k // 32, 18), np.uint8)
    out[:, :, 0:2] = d.astype(np.float16).view(np.uint8).reshape(n, k // 32, 2)
    out[:, :, 2:] = q[:, :, :16] | (q[:, :, 16:] << 4)
    return out.reshape(n, -1)


def quantize_q8_0(x: np.ndarray) -> np.ndarray:
    n, k = x.shape
    xb = x.reshape(n, k // 32, 32)
    amax = np.abs(xb).max(axis=2)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
    v = (xb * inv[..., None]).astype(np.float32)
    q = (np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))).astype(np.int8)  # round half away from zero
    out = np.empty((n, k // 32, 34), np.uint8)
    out[:, :, 0:2] = d.astype(np.float16).view(np.uint8).reshape(n, k // 32, 2)
    out[:, :, 2:] = q.view(np.uint8)
    return out.reshape(n, -1)

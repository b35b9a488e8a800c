"""Independent numpy restatement of the formats' value semantics (tables from the closed forms),
used to brute-force small cases against the C oracle."""
import numpy as np

E2M1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float64)


def _e4m3_table():
    t = np.empty(256, dtype=np.float64)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e, m = (c >> 3) & 0xF, c & 7
        if e == 15 and m == 7:
            t[c] = np.nan
        elif e == 0:
            t[c] = s * m * 2.0 ** -9
        else:
            t[c] = s * (1 + m / 8) * 2.0 ** (e - 7)
    return t


E4M3 = _e4m3_table()


def bf16_bits_to_f64(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def f32_to_bf16_f64(x32):
    """fp32 array -> the bf16-rounded values as fp64 (RNE; finite inputs)."""
    u = np.asarray(x32, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32) << 16
    return r.astype(np.uint32).view(np.float32).astype(np.float64)


def dequant_fp4(payload, scales, group):
    """[n, k/2] bytes + per-row scale bytes -> fp64 weights without the global."""
    n, half = payload.shape
    k = half * 2
    codes = np.empty((n, k), dtype=np.uint8)
    codes[:, 0::2] = payload & 0xF
    codes[:, 1::2] = payload >> 4
    w = E2M1[codes]
    if group == 16:
        s = E4M3[scales]
    else:
        s = np.where(scales == 255, np.nan, np.exp2(scales.astype(np.float64) - 127))
    return w * np.repeat(s, group, axis=1)


def dequant_fp8(payload, scales, rs, cs, strict=True, e8m0=False):
    n, k = payload.shape
    dec = E4M3[payload]
    rows = np.arange(n) >> rs
    cols = np.arange(k) >> cs
    if e8m0:
        sv = np.where(scales == 0, 2.0 ** -127, np.exp2(scales.astype(np.float64) - 127))
        sv = np.where(scales == 255, np.inf, sv)
    else:
        sv = scales.astype(np.float64)
    s = sv.reshape(-1, (k + (1 << cs) - 1) >> cs)[rows][:, cols]
    if not strict:
        return dec * s
    prod32 = (dec.astype(np.float32) * s.astype(np.float32))  # one fp32 multiply
    return f32_to_bf16_f64(prod32)


def gemv(act_bits, w64, divisor=1.0):
    return (bf16_bits_to_f64(act_bits) @ w64.T) / divisor

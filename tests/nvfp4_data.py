"""Independent numpy restatement of the NVFP4 activation quantizer's recipe (src/kernels/moe_w4a4.cu:139-236) and its
test data. Shares no code with the oracle: conversions go through value tables and midpoint searches, the arithmetic
through numpy float32 operations (one IEEE rounding each, as in the reference)."""
import numpy as np

from np_ref import bf16_bits_to_f64

E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def _e4m3_table():
    vals = []
    for c in range(0x7F):                       # 0x7F is NaN
        e, m = c >> 3, c & 7
        vals.append(m * 2.0 ** -9 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7))
    return np.array(vals)


E4M3 = _e4m3_table()


def _nearest_even_code(table, mag):
    """Index of the table value nearest to each magnitude; a tie goes to the even index; beyond the top saturates."""
    mag = np.asarray(mag, dtype=np.float64)
    idx = np.searchsorted(table, mag, side="left")          # first value >= mag
    idx = np.clip(idx, 1, len(table) - 1)
    lo, hi = table[idx - 1], table[idx]
    mid = (lo + hi) / 2
    pick_hi = (mag > mid) | ((mag == mid) & (idx % 2 == 0))
    out = np.where(pick_hi, idx, idx - 1)
    return np.where(mag >= table[-1], len(table) - 1, out).astype(np.uint8)


def e4m3_encode(v32):
    v = np.asarray(v32, dtype=np.float32).astype(np.float64)
    return (_nearest_even_code(E4M3, np.abs(v)) | np.where(np.signbit(v), 0x80, 0)).astype(np.uint8)


def e4m3_decode(codes):
    c = np.asarray(codes, dtype=np.uint8)
    return np.where(c & 0x80, -1.0, 1.0) * E4M3[np.minimum(c & 0x7F, 0x7E)]


def e2m1_encode(v32):
    v = np.asarray(v32, dtype=np.float32).astype(np.float64)
    return (_nearest_even_code(E2M1, np.abs(v)) | np.where(np.signbit(v), 8, 0)).astype(np.uint8)


def e2m1_decode(nib):
    n = np.asarray(nib, dtype=np.uint8)
    return np.where(n & 8, -1.0, 1.0) * E2M1[n & 7]


def scale_stride(k):
    return ((k // 16) + 7) // 8 * 8


def quantize_numpy(x_bits, k, static_gs=0.0):
    """(codes [rows, k/2], scales [rows, stride] with unwritten bytes 0xAA, gs [rows]) by the recipe, in numpy float32."""
    rows = x_bits.shape[0]
    x = bf16_bits_to_f64(x_bits[:, :k]).astype(np.float32)
    f = np.float32
    amax = np.abs(x).max(axis=1)
    gs = np.where(f(static_gs) > 0, f(static_gs), np.where(amax > 0, amax / (f(6.0) * f(448.0)), f(1.0))).astype(np.float32)
    xg = x.reshape(rows, k // 16, 16)
    gmax = np.abs(xg).max(axis=2)
    sb = e4m3_encode(gmax / (f(6.0) * gs[:, None]))
    bs = e4m3_decode(sb).astype(np.float32)
    dead = (gmax == 0) | (bs == 0)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = (f(1.0) / (bs * gs[:, None])).astype(np.float32)
    with np.errstate(invalid="ignore"):
        scaled = (xg * np.where(dead, f(0), q)[:, :, None]).astype(np.float32)
    nib = e2m1_encode(scaled)
    nib = np.where(dead[:, :, None], 0, nib).reshape(rows, k)
    codes = (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)
    scales = np.full((rows, scale_stride(k)), 0xAA, np.uint8)
    scales[:, :k // 16] = np.where(dead, 0, sb)
    return codes, scales, gs


def dequantize(codes, scales, gs, k):
    rows = codes.shape[0]
    nib = np.empty((rows, k), np.uint8)
    nib[:, 0::2], nib[:, 1::2] = codes & 15, codes >> 4
    return e2m1_decode(nib) * np.repeat(e4m3_decode(scales[:, :k // 16]), 16, axis=1) * np.asarray(gs, np.float64)[:, None]


def f32_to_bf16_bits(v):
    u = np.asarray(v, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def representable_rows(k, rows=33, seed=17):
    """The reference test's known-answer rows (tests/cuda/moe_w4a4_test.cu:291-303): every value on the NVFP4 grid of
    block scale 0.25 under a global of 1, every block holding its maximum 1.5 somewhere."""
    grid = np.array([0, .125, -.125, .25, -.25, .375, -.375, .5, -.5, .75, -.75, 1.0, -1.0, 1.5], np.float32)
    rng = np.random.default_rng(seed)
    x = grid[rng.integers(0, 14, (rows, k))]
    g = k // 16
    at = rng.integers(0, 16, (rows, g))
    sign = np.where(rng.integers(0, 2, (rows, g)) == 1, 1.5, -1.5).astype(np.float32)
    x.reshape(rows, g, 16)[np.arange(rows)[:, None], np.arange(g)[None, :], at] = sign
    return f32_to_bf16_bits(x)


def activation_rows(rows, k, seed, stride=None):
    """N(0, 1) rows with one value in 256 blown up twenty times (outliers, as real hidden states have)."""
    rng = np.random.default_rng(seed)
    stride = stride or k
    x = rng.normal(0, 1, (rows, stride)).astype(np.float32)
    x[rng.integers(0, 256, (rows, stride)) == 0] *= 20
    return f32_to_bf16_bits(x)


def minimax_quantize_numpy(x_bits, k):
    """The per-token dynamic producer (src/kernels/minimax_native_moe.cu:36-85) in numpy float32, reciprocals correctly
    rounded: (codes [rows, k/2], scales [rows, k/16], globals [rows])."""
    rows = x_bits.shape[0]
    f = np.float32
    x = bf16_bits_to_f64(x_bits[:, :k]).astype(np.float32)
    amax = np.abs(x).max(axis=1)
    decode = (amax * (f(1.0) / (f(6.0) * f(448.0)))).astype(np.float32)
    with np.errstate(divide="ignore"):
        encode = np.where(amax == 0, np.finfo(np.float32).max, f(1.0) / decode).astype(np.float32)
    xg = x.reshape(rows, k // 16, 16)
    gmax = np.abs(xg).max(axis=2)
    sb = e4m3_encode((encode[:, None] * (gmax * (f(1.0) / f(6.0))).astype(np.float32)).astype(np.float32))
    sv = e4m3_decode(sb).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = np.where(sv == 0, f(0), f(1.0) / (sv * (f(1.0) / encode)[:, None]).astype(np.float32)).astype(np.float32)
    nib = e2m1_encode((xg * inv[:, :, None]).astype(np.float32)).reshape(rows, k)
    codes = (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)
    return codes, sb.astype(np.uint8), decode

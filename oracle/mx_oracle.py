"""CPU oracle for the reorder-quantize -> mixed MXFP4/6/8 GEMM path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module;
it is the checker used by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py.  The product path is the HIP library and fails
loudly when that library is missing.

This is a NumPy restatement, written from the source text, of the algorithm in
the reference (all citations relative to the reference tree):

  * gather by reorder index ................ src/reorder.cu:154-158, 328-332
  * per-32 absmax .......................... src/reorder.cu:83-91, 166-169
  * power-of-two scale / E8M0 byte ......... src/reorder.cu:175-209, 349-383
  * round -> clamp -> bf16 -> element fmt .. src/reorder.cu:221-248, 399-415
  * fp4 / fp6 / fp8 packing ................ src/reorder.cu:30-33, 54-63, 250-268
  * scale-factor buffer layout ............. include/reorder.cuh:119-124,
                                             src/reorder.cu:182-185, src/fp4.cu:130-138
  * output / scale buffer sizes ............ src/bindings.cpp:85-93, 204-212
  * segment GEMM chain (alpha/beta) ........ src/gemm.cu:44-46, src/fp6.cu:178, src/fp8.cu:178

The element converters the reference calls live in NVIDIA CUTLASS (not vendored
in the reference, version unpinned); their published behaviour (OCP MX element
formats, round-to-nearest-even, saturating, sign of zero kept) is restated here.

Pins (tests/test_oracle_pins.py):
  * E4M3 rounding ........ torch.float8_e4m3fn cast (library routine)
  * E2M1 / E3M2 rounding . brute-force nearest-even search over the OCP value grid
                           versus a bit-manipulation converter in oracle/ref_scalar.c
  * scale exponent ....... closed form e = min{e : amax <= MAX*2^e}, versus the
                           literal float formula ceil(log2(amax/MAX)) of
                           oracle/ref_scalar.c over every positive finite bf16 value
  * E8M0 byte ............ torch.float8_e8m0fnu cast
  * packing .............. bit-level unpack round trip, hand-computed vectors
  * scale layout ......... injectivity, dword property, size, hand-computed offsets
  * GEMM ................. float64 brute-force dot products on tiny shapes

Parity unpinned (needs the real reference on NVIDIA Blackwell + CUTLASS; outside
every benchmark configuration's value range): NaN / Inf inputs, and blocks whose
absmax is below MAX * 2^-127 (the reference's scale leaves the bf16/E8M0 normal
range there).  This oracle defines the scale exponent as clamped to >= -127.
"""
from __future__ import annotations

import numpy as np

GROUP = 32

# element formats: name -> (exponent bits, mantissa bits, bias, max magnitude)
FORMATS = {
    "e2m1": (2, 1, 1, 6.0),     # FP4_MAX, src/reorder.cu:17
    "e3m2": (3, 2, 3, 28.0),    # FP6_MAX, src/reorder.cu:18
    "e4m3": (4, 3, 7, 448.0),   # FP8_MAX, src/reorder.cu:19
}
BITS = {"e2m1": 4, "e3m2": 6, "e4m3": 8}


# --------------------------------------------------------------------------
# element formats
# --------------------------------------------------------------------------
def format_grid(fmt: str) -> np.ndarray:
    """Magnitude of every non-negative code of `fmt` (OCP MX v1.0 tables).

    Code c = (exp << mbits) | man ; exp == 0 is subnormal.  E4M3 code 0x7f is
    NaN (no infinities in any of the three formats) and is returned as nan.
    """
    ebits, mbits, bias, _ = FORMATS[fmt]
    n = 1 << (ebits + mbits)
    out = np.empty(n, dtype=np.float64)
    for c in range(n):
        e, m = c >> mbits, c & ((1 << mbits) - 1)
        if e == 0:
            out[c] = m * 2.0 ** (1 - bias - mbits)
        else:
            out[c] = (1.0 + m * 2.0 ** -mbits) * 2.0 ** (e - bias)
    if fmt == "e4m3":
        out[0x7F] = np.nan
    return out


def rne_to_format(mag: np.ndarray, fmt: str) -> np.ndarray:
    """Round non-negative magnitudes to the nearest code of `fmt`, ties to the
    even code, saturating at the format maximum.  Brute force over the grid."""
    grid = format_grid(fmt)
    maxv = FORMATS[fmt][3]
    valid = np.where(np.isnan(grid), np.inf, grid)
    mag = np.minimum(np.asarray(mag, dtype=np.float64), maxv)
    d = np.abs(mag[..., None] - valid)
    best = d.min(axis=-1, keepdims=True)
    cand = d == best                      # one or two neighbours
    codes = np.arange(grid.size)
    even_first = np.where(cand & (codes % 2 == 0), codes, grid.size + codes)
    even_first = np.where(cand, even_first, 4 * grid.size)
    pick = even_first.min(axis=-1)
    return (pick % grid.size).astype(np.uint8)


def bf16_rne(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bf16 (ties to even), returned as float32."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32)


_LUT_CACHE: dict = {}


def integer_lut(fmt: str) -> np.ndarray:
    """LUT[|v|] for integer |v| in 0..MAX: code magnitude after the bf16 hop and
    the RNE conversion to the element format (src/reorder.cu:223-246)."""
    if fmt not in _LUT_CACHE:
        maxv = int(FORMATS[fmt][3])
        v = np.arange(maxv + 1, dtype=np.float32)
        _LUT_CACHE[fmt] = rne_to_format(bf16_rne(v).astype(np.float64), fmt)
    return _LUT_CACHE[fmt]


def decode_codes(codes: np.ndarray, fmt: str) -> np.ndarray:
    """Element codes (sign in the top bit of the 4/6/8-bit field) -> float32."""
    bits = BITS[fmt]
    grid = format_grid(fmt).astype(np.float32)
    codes = np.asarray(codes).astype(np.int64)
    mag = grid[codes & ((1 << (bits - 1)) - 1)]
    return np.where((codes >> (bits - 1)) & 1, -mag, mag).astype(np.float32)


# --------------------------------------------------------------------------
# scale
# --------------------------------------------------------------------------
def scale_exponent(amax: np.ndarray, fmt: str) -> np.ndarray:
    """e = min{e in Z : amax <= MAX * 2^e} for amax > 0, which is what
    ceil(log2(amax / MAX)) evaluates to (src/reorder.cu:180,192,204); amax == 0
    gives e = -1 (scale 0.5, src/reorder.cu:179).  Clamped below at -127."""
    amax = np.asarray(amax, dtype=np.float32)
    f, p = np.frexp(amax.astype(np.float64))          # amax = f * 2^p, f in [0.5, 1)
    # MAX = fm * 2^pm with fm in [0.5, 1)
    fm, pm = np.frexp(FORMATS[fmt][3])
    e = p - pm + (f > fm)
    e = np.maximum(e, -127)
    return np.where(amax == 0, -1, e).astype(np.int32)


def quantize_blocks(xr: np.ndarray, fmt: str):
    """xr: float32 [..., nblk, 32] (bf16-representable values, already in
    reordered order).  Returns (codes uint8 [..., nblk, 32], e8m0 uint8 [..., nblk])."""
    bits = BITS[fmt]
    maxv = FORMATS[fmt][3]
    xr = np.asarray(xr, dtype=np.float32)
    amax = np.abs(xr).max(axis=-1)
    e = scale_exponent(amax, fmt)
    # x * (1/scale): exact, scale is a power of two (src/reorder.cu:212,223)
    v = np.ldexp(xr.astype(np.float64), -e[..., None])
    mag = np.floor(np.abs(v) + 0.5)                   # roundf: half away from zero
    mag = np.minimum(mag, maxv).astype(np.int64)      # clamp (src/reorder.cu:223)
    code = integer_lut(fmt)[mag]
    sign = np.signbit(xr).astype(np.uint8)
    codes = (code | (sign << (bits - 1))).astype(np.uint8)
    return codes, (e + 127).astype(np.uint8)


# --------------------------------------------------------------------------
# packing
# --------------------------------------------------------------------------
def pack_fp4(codes: np.ndarray) -> np.ndarray:
    """[..., n] 4-bit codes -> [..., n/2] bytes, even element in the low nibble
    (src/reorder.cu:30-33,243-246)."""
    c = np.asarray(codes, dtype=np.uint8)
    return np.ascontiguousarray((c[..., 0::2] & 0xF) | ((c[..., 1::2] & 0xF) << 4))


def unpack_fp4(b: np.ndarray) -> np.ndarray:
    b = np.asarray(b, dtype=np.uint8)
    out = np.empty(b.shape[:-1] + (b.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = b & 0xF
    out[..., 1::2] = b >> 4
    return out


def pack_fp6(codes: np.ndarray) -> np.ndarray:
    """[..., n] 6-bit codes -> [..., 3n/4] bytes, little-endian bit stream
    (src/reorder.cu:54-63)."""
    c = np.asarray(codes, dtype=np.uint8) & 0x3F
    v0, v1, v2, v3 = (c[..., i::4].astype(np.uint16) for i in range(4))
    out = np.empty(c.shape[:-1] + (c.shape[-1] // 4 * 3,), dtype=np.uint8)
    out[..., 0::3] = (v0 | ((v1 & 0x03) << 6)) & 0xFF
    out[..., 1::3] = ((v1 >> 2) | ((v2 & 0x0F) << 4)) & 0xFF
    out[..., 2::3] = ((v2 >> 4) | (v3 << 2)) & 0xFF
    return out


def unpack_fp6(b: np.ndarray) -> np.ndarray:
    b = np.asarray(b, dtype=np.uint8).astype(np.uint32)
    w = b[..., 0::3] | (b[..., 1::3] << 8) | (b[..., 2::3] << 16)
    out = np.empty(b.shape[:-1] + (b.shape[-1] // 3 * 4,), dtype=np.uint8)
    for i in range(4):
        out[..., i::4] = (w >> (6 * i)) & 0x3F
    return out


# --------------------------------------------------------------------------
# scale-factor buffer layout
# --------------------------------------------------------------------------
def sf_offset(r, kb, kseg: int):
    """Byte offset of the scale of (row r, 32-element block kb) inside one
    segment's scale buffer: 128-row x 4-block atoms of 512 bytes, K atoms
    fastest (include/reorder.cuh:119-124; coordinates src/reorder.cu:182-185)."""
    r = np.asarray(r, dtype=np.int64)
    kb = np.asarray(kb, dtype=np.int64)
    katoms = (kseg + 127) // 128
    return ((r // 128) * katoms + kb // 4) * 512 + (r % 32) * 16 + ((r // 32) % 4) * 4 + (kb % 4)


def sf_bytes(rows: int, kseg: int, operand: str) -> int:
    """Size of a scale buffer.  operand 'a': (rows/128 + 1)*128*kseg/32
    (src/bindings.cpp:91-93); operand 'b': rows*kseg/32 (src/bindings.cpp:210-212);
    never less than the layout itself spans."""
    span = ((rows + 127) // 128) * ((kseg + 127) // 128) * 512
    ref = (rows // 128 + 1) * 128 * kseg // 32 if operand == "a" else rows * kseg // 32
    return max(ref, span)


def sf_scatter(e8m0: np.ndarray, kseg: int, operand: str, fill: int = 0) -> np.ndarray:
    """Logical [rows, kseg/32] scale bytes -> laid-out buffer."""
    rows, nb = e8m0.shape
    buf = np.full(sf_bytes(rows, kseg, operand), fill, dtype=np.uint8)
    if nb:
        r, kb = np.meshgrid(np.arange(rows), np.arange(nb), indexing="ij")
        buf[sf_offset(r, kb, kseg)] = e8m0
    return buf


def sf_gather(buf: np.ndarray, rows: int, kseg: int) -> np.ndarray:
    """Laid-out buffer -> logical [rows, kseg/32] scale bytes."""
    nb = kseg // GROUP
    if nb == 0 or rows == 0:
        return np.zeros((rows, nb), dtype=np.uint8)
    r, kb = np.meshgrid(np.arange(rows), np.arange(nb), indexing="ij")
    return np.asarray(buf, dtype=np.uint8)[sf_offset(r, kb, kseg)]


# --------------------------------------------------------------------------
# the two quantizers
# --------------------------------------------------------------------------
def _segments(kn, ks, ko):
    assert kn % GROUP == 0 and ks % GROUP == 0 and ko % GROUP == 0
    return (0, kn), (kn, kn + ks), (kn + ks, kn + ks + ko)


def reorder_quantize_x(x: np.ndarray, idx: np.ndarray, kn: int, ks: int, ko: int) -> dict:
    """Activation path (src/reorder.cu:94-269).  x float32 [M, K] holding bf16
    values; idx integer [K].  Returns packed codes, laid-out scale buffers and the
    logical (unpacked) codes / scale bytes."""
    x = np.asarray(x, dtype=np.float32)
    m = x.shape[0]
    xr = np.ascontiguousarray(x[:, np.asarray(idx, dtype=np.int64)])
    out = {}
    for name, fmt, (lo, hi), pack in zip(
        ("n", "s", "o"), ("e2m1", "e3m2", "e4m3"), _segments(kn, ks, ko),
        (pack_fp4, pack_fp6, lambda c: c.copy()),
    ):
        kseg = hi - lo
        codes, e8 = quantize_blocks(xr[:, lo:hi].reshape(m, kseg // GROUP, GROUP), fmt)
        codes = codes.reshape(m, kseg)
        out["q" + name] = pack(codes)
        out["sf" + name] = sf_scatter(e8, kseg, "a")
        out["codes_" + name] = codes
        out["e8m0_" + name] = e8
    return out


def reorder_quantize_w(w: np.ndarray, idx: np.ndarray, kn: int, ks: int, ko: int) -> dict:
    """Weight path (src/reorder.cu:271-432): same gather and scale rule, every
    segment quantized to E2M1."""
    w = np.asarray(w, dtype=np.float32)
    n = w.shape[0]
    wr = np.ascontiguousarray(w[:, np.asarray(idx, dtype=np.int64)])
    out = {}
    for name, (lo, hi) in zip(("n", "s", "o"), _segments(kn, ks, ko)):
        kseg = hi - lo
        codes, e8 = quantize_blocks(wr[:, lo:hi].reshape(n, kseg // GROUP, GROUP), "e2m1")
        codes = codes.reshape(n, kseg)
        out["q" + name] = pack_fp4(codes)
        out["sf" + name] = sf_scatter(e8, kseg, "b")
        out["codes_" + name] = codes
        out["e8m0_" + name] = e8
    return out


# --------------------------------------------------------------------------
# dequantize + GEMM
# --------------------------------------------------------------------------
def dequantize(codes: np.ndarray, e8m0: np.ndarray, fmt: str) -> np.ndarray:
    """codes [R, kseg] + scale bytes [R, kseg/32] -> float32 [R, kseg]."""
    r, kseg = codes.shape
    vals = decode_codes(codes, fmt).reshape(r, kseg // GROUP, GROUP)
    scale = np.ldexp(np.float32(1), e8m0.astype(np.int32) - 127).astype(np.float32)
    return (vals * scale[..., None]).reshape(r, kseg)


def dequantize_x(q: dict) -> np.ndarray:
    """Dequantized activations in reordered channel order, float32 [M, K]."""
    return np.concatenate(
        [dequantize(q["codes_" + n], q["e8m0_" + n], f)
         for n, f in (("n", "e2m1"), ("s", "e3m2"), ("o", "e4m3"))], axis=1)


def dequantize_w(q: dict) -> np.ndarray:
    return np.concatenate(
        [dequantize(q["codes_" + n], q["e8m0_" + n], "e2m1") for n in ("n", "s", "o")], axis=1)


def mixed_matmul(qx: dict, qw: dict, chain_bf16: bool = False) -> np.ndarray:
    """fp32 result of A.B^T over the three segments (float64 accumulation, cast
    to float32).  chain_bf16=True reproduces the reference's bf16 round trip of D
    between the segment GEMMs (src/gemm.cu:44-46: beta = 0, 1, 1) and returns the
    bf16 values as float32."""
    acc = None
    for n, f in (("n", "e2m1"), ("s", "e3m2"), ("o", "e4m3")):
        if qx["codes_" + n].shape[1] == 0:
            continue
        a = dequantize(qx["codes_" + n], qx["e8m0_" + n], f).astype(np.float64)
        b = dequantize(qw["codes_" + n], qw["e8m0_" + n], "e2m1").astype(np.float64)
        seg = a @ b.T
        if chain_bf16:
            prev = 0.0 if acc is None else acc.astype(np.float64)
            acc = bf16_rne((seg + prev).astype(np.float32))
        else:
            acc = seg if acc is None else acc + seg
    if acc is None:
        return np.zeros((qx["codes_n"].shape[0], qw["codes_n"].shape[0]), dtype=np.float32)
    return acc.astype(np.float32)


def fake_quant_linear(x, w, idx, kn, ks, ko):
    """End-to-end reference semantics on the host: quantize X and W, dequantize,
    fp32 matmul, bf16 output (as float32)."""
    qx = reorder_quantize_x(x, idx, kn, ks, ko)
    qw = reorder_quantize_w(w, idx, kn, ks, ko)
    return bf16_rne(mixed_matmul(qx, qw))


def calibrate_reorder_index(x_bits):
    """Reorder index of a bf16 sample given as uint16 bit patterns [M, K]: channels by ascending
    per-channel max |x|, ties by channel number, int16 (main.py:31-33 of the reference:
    torch.max(torch.abs(X), dim=0).values -> torch.sort ascending -> int16; torch leaves the order
    of ties open, here it is fixed).  For finite values the bf16 bit pattern with the sign cleared
    orders like |x|, so no float conversion is needed."""
    mag = (np.asarray(x_bits, dtype=np.uint16) & 0x7FFF).max(axis=0).astype(np.uint32)
    return np.argsort(mag, kind="stable").astype(np.int16)


def rmsnorm_bf16(x_bits, gamma_bits, eps):
    """RMSNorm of bf16 rows x[M, K] with bf16 weight gamma[K], as bf16 bit patterns -- the
    arithmetic the usual fp32 implementation spells out (to fp32, mean of squares, rsqrt, back to
    bf16, times the weight), with the reduction and the reciprocal square root pinned so that the
    result does not depend on who computes it:
        var = fl32( (sum of x^2 in float64) / K );  r = fl32( 1 / sqrt( fl32(var + eps) ) )  in float64;
        y   = bf16( gamma * bf16( x * r ) ), both products in float32.
    The reference has no normalisation layer: this is the layer in front of a quantized linear."""
    x = (np.asarray(x_bits, np.uint16).astype(np.uint32) << 16).view(np.float32)
    g = (np.asarray(gamma_bits, np.uint16).astype(np.uint32) << 16).view(np.float32)
    k = x.shape[1]
    ss = (x.astype(np.float64) ** 2).sum(axis=1)
    var = (ss / np.float64(k)).astype(np.float32)
    t = (var + np.float32(eps)).astype(np.float32)
    r = (1.0 / np.sqrt(t.astype(np.float64))).astype(np.float32)
    h = bf16_rne((x * r[:, None]).astype(np.float32))
    y = bf16_rne((g[None, :] * h).astype(np.float32))
    return (y.view(np.uint32) >> 16).astype(np.uint16)

"""GPU parity tests: the HIP path, called through the C-ABI, against the CPU
oracle on the same seeded inputs.  Codes and scales are bit-exact; GEMM output is
within 1 bf16 ulp of the bf16-rounded float64 product of the dequantized
operands (plus an accumulation-order allowance stated below)."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as mo
from oracle import scalar as sc
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def abi():
    from mixedgemm_amd import abi as a
    a.lib()                      # raises if the HIP library is missing
    return a


def _say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------ quantizers
QUANT_SHAPES = [
    # rows, KN, KS, KO
    (4, 128, 0, 0), (4, 0, 128, 0), (4, 0, 0, 128),
    (5, 64, 96, 96), (3, 32, 32, 32), (130, 2560, 1408, 128), (114, 2560, 896, 128),
    (7, 3072, 1920, 128), (9, 8960, 4928, 448), (2, 12288, 6400, 256), (5, 7680, 4224, 384),
    (6, 8704, 4736, 384), (1, 4096, 0, 0), (257, 256, 128, 128), (3, 20480, 8192, 4064),
]


def _quant_inputs(rows, k, seed):
    x = H.make_activations(rows, k, seed, n_out=max(1, k // 32))
    idx = H.random_index(k, seed + 1)
    return x, idx


@pytest.mark.parametrize("rows,kn,ks,ko", QUANT_SHAPES)
@pytest.mark.parametrize("which", ["x", "w"])
def test_reorder_quantize_matches_oracle(abi, which, rows, kn, ks, ko):
    k = kn + ks + ko
    _say("quant", which, rows, kn, ks, ko)
    x, idx = _quant_inputs(rows, k, 100 + rows)
    if which == "x":
        got = abi.reorder_quantize_x(x.to(DEV), idx.to(DEV), kn, ks, ko)
        want = sc.quantize_x(H.bf16_bits(x), idx.numpy(), kn, ks, ko)
    else:
        got = abi.reorder_quantize_w(x.to(DEV), idx.to(DEV), kn, ks, ko)
        want = sc.quantize_w(H.bf16_bits(x), idx.numpy(), kn, ks, ko)
    torch.cuda.synchronize()
    H.assert_quant_equal(got, want, rows, (kn, ks, ko), what=f"{which} {rows}x{k}")


def _adversarial(k):
    rows = []
    z = np.zeros(k, np.float32)
    rows.append(z.copy())
    r = z.copy(); r[:] = -0.0; rows.append(r)
    r = z.copy(); r[::32] = 6.0; r[1::32] = -0.25; r[2::32] = 2.5; r[3::32] = -4.5; r[4::32] = 5.0; r[5::32] = 0.5; r[6::32] = -1.5; r[7::32] = 3.5; rows.append(r)
    r = z.copy(); r[::32] = 28.0; r[1::32] = 9.0; r[2::32] = -13.0; r[3::32] = 26.0; r[4::32] = 10.5; r[5::32] = -0.4375; r[6::32] = 11.0; r[7::32] = 15.0; r[8::32] = 18.0; r[9::32] = -22.0; rows.append(r)
    r = z.copy(); r[::32] = 448.0; r[1::32] = 273.0; r[2::32] = -431.0; r[3::32] = 17.0; r[4::32] = 272.5; r[5::32] = 303.0; r[6::32] = 337; r[7::32] = -367; r[8::32] = 401; rows.append(r)
    r = z.copy(); r[::32] = 6.0 * 2.0 ** -20; r[1::32] = -5.0 * 2.0 ** -20; rows.append(r)
    r = z.copy(); r[::32] = 3.0e38; r[1::32] = -1.0e38; rows.append(r)
    r = z.copy(); r[::32] = 6.03125; r[7::32] = 3.0; rows.append(r)
    r = z.copy(); r[::32] = 2.0 ** -100; r[1::32] = -1.5 * 2.0 ** -101; rows.append(r)
    # every integer magnitude of each format as x with the block max pinned at MAX
    for maxv in (6, 28, 448):
        for start in range(0, maxv + 1, 30):
            r = z.copy()
            for b in range(k // 32):
                vals = np.arange(start, min(start + 30, maxv + 1), dtype=np.float32)
                r[32 * b] = maxv
                r[32 * b + 1: 32 * b + 1 + vals.size] = vals * (-1) ** b
                r[32 * b + 31] = -0.5
            rows.append(r)
    return torch.from_numpy(np.stack(rows)).to(torch.bfloat16)


@pytest.mark.parametrize("kn,ks,ko", [(128, 128, 128), (2560, 1408, 128)])
def test_reorder_quantize_adversarial_blocks(abi, kn, ks, ko):
    k = kn + ks + ko
    x = _adversarial(k)
    idx = torch.arange(k, dtype=torch.int16)
    rows = x.shape[0]
    _say("adversarial", rows, k)
    for which, fn, ofn in (("x", abi.reorder_quantize_x, sc.quantize_x), ("w", abi.reorder_quantize_w, sc.quantize_w)):
        got = fn(x.to(DEV), idx.to(DEV), kn, ks, ko)
        torch.cuda.synchronize()
        H.assert_quant_equal(got, ofn(H.bf16_bits(x), idx.numpy(), kn, ks, ko), rows, (kn, ks, ko), what=which)


def test_denormal_blocks_follow_the_clamped_scale_rule(abi):
    """Blocks below MAX*2^-127 are outside the reference's pinned behaviour; the
    library follows the oracle's definition (scale exponent clamped at -127)."""
    k = 384
    x = torch.zeros(4, k, dtype=torch.float32)
    x[0, ::32] = 2.0 ** -126
    x[1, ::32] = 2.0 ** -130
    x[1, 1::32] = -(2.0 ** -133)
    x[2, ::32] = 6 * 2.0 ** -127
    x[3, ::32] = 2.0 ** -120
    x[3, 1::32] = 2.0 ** -131
    x = x.to(torch.bfloat16)
    idx = torch.arange(k, dtype=torch.int16)
    got = abi.reorder_quantize_x(x.to(DEV), idx.to(DEV), 128, 128, 128)
    torch.cuda.synchronize()
    H.assert_quant_equal(got, sc.quantize_x(H.bf16_bits(x), idx.numpy(), 128, 128, 128), 4, (128, 128, 128))


def test_config1_full_size_bit_exact(abi):
    m, _, k, kn, ks, ko = H.CONFIGS["c1"]
    _say("c1 full size")
    x = H.make_activations(m, k, 1235)
    idx = H.random_index(k, 4321)
    got = abi.reorder_quantize_x(x.to(DEV), idx.to(DEV), kn, ks, ko)
    torch.cuda.synchronize()
    H.assert_quant_equal(got, sc.quantize_x(H.bf16_bits(x), idx.numpy(), kn, ks, ko), m, (kn, ks, ko), what="c1")


# ------------------------------------------------------------------ GEMM
def _oracle_operands(x, w, idx, kn, ks, ko):
    qx = mo.reorder_quantize_x(H.bf16_f32(x), idx.numpy(), kn, ks, ko)
    qw = mo.reorder_quantize_w(H.bf16_f32(w), idx.numpy(), kn, ks, ko)
    return qx, qw


def _to_dev(q):
    return [torch.from_numpy(q[n]).to(DEV) for n in ("qn", "qs", "qo", "sfn", "sfs", "sfo")]


def _check_gemm(d, qx, qw, what):
    """|d - bf16(ref)| <= 1 bf16 ulp, where ref is the float64 product of the
    dequantized operands; sums that cancel get an allowance of 2^-20 of the sum of
    absolute products (fp32 accumulation order)."""
    ref = mo.mixed_matmul(qx, qw)
    a = np.abs(mo.dequantize_x(qx)).astype(np.float64)
    b = np.abs(mo.dequantize_w(qw)).astype(np.float64)
    slack = (a @ b.T) * 2.0 ** -20
    got = d.float().cpu().numpy()
    err = np.abs(got - mo.bf16_rne(ref))
    tol = H.bf16_ulp(ref) + slack
    bad = err > tol
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} outside 1 bf16 ulp; max err {err.max()} at {np.unravel_index(err.argmax(), err.shape)}"
    # and within rtol 2e-3 of the fp32 reference up to the bf16 rounding of the output itself
    rel = np.abs(got - ref) <= 2e-3 * np.abs(ref) + 0.5 * H.bf16_ulp(ref) + slack
    assert rel.all(), what


GEMM_SHAPES = [
    # M, N, KN, KS, KO
    (16, 16, 128, 0, 0), (16, 16, 0, 128, 0), (16, 16, 0, 0, 128),
    (16, 64, 128, 128, 128), (8, 64, 256, 128, 128), (33, 80, 64, 96, 32),
    (64, 128, 512, 384, 128), (114, 256, 2560, 896, 128), (128, 512, 2560, 1408, 128),
    (20, 64, 448, 224, 64), (1, 16, 32, 32, 32),
    # decode kernel (M <= 16): ragged N, partial K steps, more K steps than one pass keeps in flight
    (8, 200, 96, 160, 64), (3, 1000, 2560, 1408, 128), (16, 48, 8192, 4096, 1024), (5, 40, 0, 4928, 448),
    # 128 tokens x 256 features and whole 128-wide K stages (the decode kernel with two token groups per workgroup, or 256 x 128 tiles where they are estimated faster)
    (128, 256, 256, 0, 0), (128, 256, 0, 256, 0), (128, 256, 0, 0, 128), (128, 256, 128, 0, 128),
    (256, 512, 384, 256, 128), (128, 256, 2560, 1408, 128), (384, 768, 1280, 640, 128),
    # whole tiles with all three segments: the one-workgroup-per-CU kernel
    (256, 256, 128, 128, 128), (512, 256, 256, 384, 128), (256, 768, 2560, 1408, 128), (512, 512, 640, 256, 256),
    # the same with at least three 128-wide stages in the first two segments (segment-boundary copies compiled in)
    (256, 256, 384, 384, 384), (512, 256, 512, 384, 128), (256, 512, 384, 512, 256),
    # segments that end 32, 64 or 96 elements past their last whole 128-wide stage
    (256, 256, 448, 416, 224), (256, 512, 2240, 1248, 448), (512, 256, 160, 480, 352),
    # 17 to 255 tokens: ragged M and N, partial K steps (skinny kernel), an empty segment
    (17, 48, 256, 128, 128), (32, 200, 96, 160, 64), (50, 40, 2560, 1408, 128), (64, 64, 0, 4928, 448),
    (100, 256, 448, 224, 64), (128, 4096, 2560, 1408, 128), (255, 272, 128, 128, 128), (200, 1000, 640, 256, 256),
    # ragged token counts: the last 256-row tile stores only part of its rows
    (300, 512, 2560, 1408, 128), (257, 256, 384, 384, 384), (767, 256, 448, 416, 224),
    # plans without E3M2 and / or E4M3 activations on the whole-tile kernel (fragments pass to the next segment that exists)
    (256, 256, 512, 0, 0), (512, 512, 128, 0, 0), (300, 256, 384, 0, 128), (256, 512, 1024, 0, 256), (256, 256, 384, 256, 0),
    (300, 512, 2560, 1536, 0), (1000, 256, 4096, 0, 0), (256, 256, 512, 0, 384), (256, 256, 384, 128, 0),
    # feature counts that are not whole 256-feature tiles (multiples of 8): the last tile's lanes read the last
    # weight row again and store only the pieces that exist
    (300, 1000, 2560, 1408, 128), (256, 264, 384, 384, 384), (512, 136, 448, 416, 224), (700, 8, 128, 128, 128),
    (256, 392, 512, 0, 0), (384, 648, 384, 0, 128),
    # plans without E2M1 activations on the whole-tile kernel: pure E3M2 x E2M1 and E4M3 x E2M1 products (the reference's
    # matmul_host6 / matmul_host8 alone), E3M2 + E4M3 with and without three stages in the first of them; and plans
    # whose first segment is shorter than three stages next to an empty one (run-time segment-boundary copies)
    (256, 256, 0, 256, 0), (512, 256, 0, 1024, 0), (300, 264, 0, 128, 0), (256, 256, 0, 0, 128), (256, 512, 0, 0, 640),
    (256, 256, 0, 384, 128), (300, 512, 0, 512, 384), (384, 256, 0, 256, 128), (256, 256, 0, 128, 256),
    (256, 256, 256, 0, 0), (256, 512, 128, 0, 128), (256, 256, 256, 128, 0), (512, 256, 128, 256, 0),
]


# decode kernel (up to 16 tokens, whole 128-wide steps): one and two feature groups per workgroup, ragged N inside
# and across groups of 128 rows, an empty segment, a single token, K beyond one round of steps per wave
DECODE_SHAPES = [
    (8, 14336, 2560, 1408, 128), (1, 4096, 2560, 1408, 128), (16, 512, 384, 256, 128), (7, 200, 128, 128, 128),
    (8, 8200, 256, 128, 0), (3, 1000, 2560, 1408, 128), (12, 136, 0, 384, 128), (8, 12288, 1280, 0, 256),
    (2, 9000, 4096, 2048, 512), (16, 8192, 128, 0, 0),
    # wide tile-major layers: four feature groups per workgroup; 16 tokens, and K beyond the first two rounds
    (16, 12288, 384, 256, 128), (5, 14336, 8960, 4928, 448),
    # a last K step of 1, 2, 3 blocks of 32 in every segment; segments shorter than a step; long K whose LDS image
    # needs a CU's whole LDS (and fewer feature groups per workgroup for 16 tokens)
    (8, 512, 416, 480, 160), (16, 768, 160, 224, 352), (4, 1024, 480, 448, 192), (9, 520, 64, 96, 32),
    (8, 4096, 8960, 4928, 448), (16, 4096, 7680, 4224, 384), (1, 3584, 11776, 6560, 608),
]


@pytest.mark.parametrize("m,n,kn,ks,ko", DECODE_SHAPES)
@pytest.mark.parametrize("tiled", [False, True])
def test_decode_kernel_matches_oracle(abi, m, n, kn, ks, ko, tiled):
    k = kn + ks + ko
    _say("decode", m, n, kn, ks, ko, "tiled" if tiled else "row-major")
    if tiled and not abi.weights_tileable(n, kn, ks, ko):
        pytest.skip("shape cannot be tiled")
    x = H.make_activations(m, k, 17 + m + n, n_out=max(1, k // 32))
    w = H.make_weights(n, k, 19 + m + n)
    idx = H.absmax_sort_index(x)
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    a, b = _to_dev(qx), _to_dev(qw)
    if tiled:
        b = list(abi.tile_weights(*b[:3])) + b[3:]
    d = abi.matmul(a[0], b[0], a[1], b[1], a[2], b[2], a[3], b[3], a[4], b[4], a[5], b[5], w_tiled=tiled)
    torch.cuda.synchronize()
    _check_gemm(d, qx, qw, f"decode {m}x{n}x{k}")


# 17 to 255 tokens with whole 128-wide steps: the decode kernel with two token groups (32 tokens) per workgroup where
# the tokens' codes fit the LDS, one to four feature groups per workgroup, ragged token and feature counts, an empty
# segment, a token count whose last workgroup has a single token group; K = 14336 does not fit (skinny kernel)
SMALL_M_SHAPES = [
    (128, 4096, 2560, 1408, 128), (32, 512, 2560, 1408, 128), (100, 4096, 2560, 1408, 128), (255, 512, 384, 256, 128),
    (40, 14336, 2560, 1408, 128), (64, 256, 0, 384, 128), (130, 1000, 1280, 0, 256), (17, 264, 128, 128, 128),
    (49, 2048, 512, 0, 0), (200, 768, 2560, 1408, 128), (33, 4096, 8960, 4928, 448),
    (32, 512, 416, 480, 160), (64, 1024, 160, 224, 352), (100, 768, 480, 448, 192),
]


@pytest.mark.parametrize("m,n,kn,ks,ko", SMALL_M_SHAPES)
@pytest.mark.parametrize("tiled", [False, True])
def test_small_batches_match_oracle(abi, m, n, kn, ks, ko, tiled):
    k = kn + ks + ko
    _say("small batch", m, n, kn, ks, ko, "tiled" if tiled else "row-major")
    if tiled and not abi.weights_tileable(n, kn, ks, ko):
        pytest.skip("shape cannot be tiled")
    x = H.make_activations(m, k, 27 + m + n, n_out=max(1, k // 32))
    w = H.make_weights(n, k, 29 + m + n)
    idx = H.absmax_sort_index(x)
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    a, b = _to_dev(qx), _to_dev(qw)
    if tiled:
        b = list(abi.tile_weights(*b[:3])) + b[3:]
    d = abi.matmul(a[0], b[0], a[1], b[1], a[2], b[2], a[3], b[3], a[4], b[4], a[5], b[5], w_tiled=tiled)
    torch.cuda.synchronize()
    _check_gemm(d, qx, qw, f"small batch {m}x{n}x{k}")
    # exact-size activation buffers: nothing is read past the last token's codes
    tight = [t.clone() for t in a]
    d2 = abi.matmul(tight[0], b[0], tight[1], b[1], tight[2], b[2], tight[3], b[3], tight[4], b[4], tight[5], b[5], w_tiled=tiled)
    torch.cuda.synchronize()
    assert torch.equal(d, d2)


@pytest.mark.parametrize("m,n,kn,ks,ko", GEMM_SHAPES)
def test_mixed_gemm_matches_oracle(abi, m, n, kn, ks, ko):
    k = kn + ks + ko
    _say("gemm", m, n, kn, ks, ko)
    x = H.make_activations(m, k, 7 + m + n, n_out=max(1, k // 32))
    w = H.make_weights(n, k, 9 + m + n)
    idx = H.absmax_sort_index(x)
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    a, b = _to_dev(qx), _to_dev(qw)
    d = abi.matmul(a[0], b[0], a[1], b[1], a[2], b[2], a[3], b[3], a[4], b[4], a[5], b[5])
    torch.cuda.synchronize()
    _check_gemm(d, qx, qw, f"gemm {m}x{n}x{k}")


# More than 128 whole tiles: 256 x 256 tiles (smaller problems run 256 x 128).  One plan per kernel family: all three
# segments with a last segment of 1, 2 and 3 stages (the kernels are compiled per length of the last segment),
# segments with a remainder, and the plans with an empty segment.
BIG_TILE_SHAPES = [
    (2304, 3840, 384, 384, 128), (2304, 3840, 384, 384, 256), (2304, 3840, 384, 384, 384), (2304, 3840, 448, 416, 224),
    (2304, 3840, 512, 0, 0), (2304, 3840, 384, 128, 0), (2304, 3840, 384, 256, 0), (2304, 3840, 384, 0, 128),
    (2304, 3840, 384, 0, 384), (2100, 3848, 384, 384, 128),
    # plans without E2M1 activations, and two-segment plans with a short first segment (tile-major weights as well)
    (2304, 3840, 0, 512, 0), (2304, 3840, 0, 0, 256), (2304, 3840, 0, 384, 128), (2304, 3840, 0, 256, 256), (2304, 3840, 256, 0, 128),
    # 1, 2 and 3 blocks of 32 past the whole stages in every segment (computed ahead of the K loop, absent K halves
    # skipped), with and without compiled-in segment boundaries, ragged tokens and features
    (2304, 3840, 416, 480, 160), (2304, 3840, 480, 448, 192), (2304, 3840, 160, 224, 352), (2100, 3848, 480, 448, 192),
    # more whole tiles than CUs with a last round on at most half of them: those tiles run as half tiles in the same
    # launch (272 = 256 + 16 tiles; a last segment of 1, 2, 3 stages; blocks past the whole stages; ragged tokens whose
    # last tile has no lower half; features that are not whole tiles)
    (4352, 4096, 384, 384, 128), (4352, 4096, 384, 384, 256), (4352, 4096, 384, 384, 384), (4352, 4096, 448, 416, 224),
    (4200, 4096, 384, 384, 128), (4300, 4104, 448, 416, 224),
    # launches of at most one tile per CU whose tile counts divide among the 8 XCDs as rectangles of tiles
    # (8 x 8, 16 x 12 and 8 x 16 tiles of 256 x 128; 16 x 8 tiles of 256 x 256), ragged tokens among them
    (1024, 2048, 384, 384, 128), (1536, 4096, 384, 384, 256), (2000, 2048, 384, 128, 0), (2048, 4096, 256, 128, 128),
]


@pytest.mark.parametrize("m,n,kn,ks,ko", BIG_TILE_SHAPES)
def test_whole_tile_kernel_with_256_token_tiles(abi, m, n, kn, ks, ko):
    k = kn + ks + ko
    _say("gemm, 256 x 256 tiles", m, n, kn, ks, ko)
    x = H.make_activations(m, k, 41 + m + n, n_out=max(1, k // 32))
    w = H.make_weights(n, k, 43 + m + n)
    idx = H.absmax_sort_index(x)
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    a, b = _to_dev(qx), _to_dev(qw)
    d = abi.matmul(a[0], b[0], a[1], b[1], a[2], b[2], a[3], b[3], a[4], b[4], a[5], b[5])
    torch.cuda.synchronize()
    _check_gemm(d, qx, qw, f"gemm {m}x{n}x{k}")
    if abi.weights_tileable(n, kn, ks, ko):
        bt = list(abi.tile_weights(*b[:3])) + b[3:]
        dt = abi.matmul(a[0], bt[0], a[1], bt[1], a[2], bt[2], a[3], bt[3], a[4], bt[4], a[5], bt[5], w_tiled=True)
        torch.cuda.synchronize()
        assert torch.equal(d, dt)


@pytest.mark.parametrize("seg", ["n", "s", "o"])
def test_gemm_operand_bit_order_one_hot(abi, seg):
    """A single non-zero activation code at (row, k) against weights whose code
    depends on (n, k): the output row must equal the decoded products, which pins
    the element order inside the packed MFMA operands."""
    m, n, kseg = 16, 32, 128
    fmt = {"n": "e2m1", "s": "e3m2", "o": "e4m3"}[seg]
    splits = {"n": (kseg, 0, 0), "s": (0, kseg, 0), "o": (0, 0, kseg)}[seg]
    rng = np.random.default_rng(5)
    wcodes = rng.integers(0, 16, (n, kseg), dtype=np.uint8)
    we8 = rng.integers(120, 130, (n, kseg // 32), dtype=np.uint8)
    for trial in range(12):
        row, kk = int(rng.integers(0, m)), int(rng.integers(0, kseg))
        code = int(rng.integers(1, 1 << (mo.BITS[fmt] - 1)))
        if fmt == "e4m3" and (code & 0x7F) == 0x7F:
            code = 0x7E
        xcodes = np.zeros((m, kseg), np.uint8)
        xcodes[row, kk] = code
        xe8 = rng.integers(120, 130, (m, kseg // 32), dtype=np.uint8)
        qx = {f"codes_{s}": np.zeros((m, 0), np.uint8) for s in "nso"}
        qx.update({f"e8m0_{s}": np.zeros((m, 0), np.uint8) for s in "nso"})
        qw = {f"codes_{s}": np.zeros((n, 0), np.uint8) for s in "nso"}
        qw.update({f"e8m0_{s}": np.zeros((n, 0), np.uint8) for s in "nso"})
        qx["codes_" + seg], qx["e8m0_" + seg] = xcodes, xe8
        qw["codes_" + seg], qw["e8m0_" + seg] = wcodes, we8
        pack = {"n": mo.pack_fp4, "s": mo.pack_fp6, "o": lambda c: c}[seg]
        empty = lambda r: torch.zeros((r, 0), dtype=torch.uint8, device=DEV)
        sfe = torch.zeros(0, dtype=torch.uint8, device=DEV)
        ops = {s: [empty(m), empty(n), sfe, sfe] for s in "nso"}
        ops[seg] = [torch.from_numpy(pack(xcodes)).to(DEV), torch.from_numpy(mo.pack_fp4(wcodes)).to(DEV),
                    torch.from_numpy(mo.sf_scatter(xe8, kseg, "a")).to(DEV),
                    torch.from_numpy(mo.sf_scatter(we8, kseg, "b")).to(DEV)]
        d = abi.matmul(ops["n"][0], ops["n"][1], ops["s"][0], ops["s"][1], ops["o"][0], ops["o"][1],
                       ops["n"][2], ops["n"][3], ops["s"][2], ops["s"][3], ops["o"][2], ops["o"][3])
        torch.cuda.synchronize()
        want = mo.bf16_rne(mo.mixed_matmul(qx, qw))
        np.testing.assert_array_equal(d.float().cpu().numpy(), want, err_msg=f"{seg} trial {trial} row {row} k {kk}")


@pytest.mark.parametrize("m,n,kn,ks,ko", [
    (96, 256, 2560, 1408, 128),
    # ragged token counts: the last 256-row tile reads rows past M from the padded buffers and does not write them
    (300, 512, 2560, 1408, 128), (130, 2560, 384, 384, 384), (1000, 256, 448, 416, 224), (255, 4096, 2560, 896, 128),
    (70, 14336, 2560, 1408, 128),
])
def test_fused_linear_equals_quantize_then_gemm(abi, m, n, kn, ks, ko):
    _say("fused", m, n, kn, ks, ko)
    k = kn + ks + ko
    x = H.make_activations(m, k, 50)
    w = H.make_weights(n, k, 51)
    idx = H.absmax_sort_index(x)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    aq = abi.reorder_quantize_x(xd, idd, kn, ks, ko)
    d1 = abi.matmul(aq[0], bq[0], aq[1], bq[1], aq[2], bq[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5])
    d2 = abi.fused_linear(xd, idd, bq[0], bq[1], bq[2], bq[3], bq[4], bq[5], kn, ks, ko)
    # exact-size activation buffers (no room past M): the last tile's lanes read no row past M
    tight = [t.clone() for t in aq]
    d3 = abi.matmul(tight[0], bq[0], tight[1], bq[1], tight[2], bq[2], tight[3], bq[3], tight[4], bq[4], tight[5], bq[5])
    torch.cuda.synchronize()
    assert torch.equal(d1, d2)
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    _check_gemm(d2, qx, qw, "fused")
    _check_gemm(d3, qx, qw, "exact-size buffers")


def test_config0_end_to_end(abi):
    """Config 0 (single linear, M=128, K=N=4096) through the whole path, against
    the host fake-quant reference semantics."""
    m, n, k, kn, ks, ko = H.CONFIGS["c0"]
    _say("c0 end to end")
    x = H.make_activations(m, k, 1234)
    w = H.make_weights(n, k, 2234)
    idx = H.absmax_sort_index(x)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    d = abi.fused_linear(xd, idd, *bq, kn, ks, ko)
    torch.cuda.synchronize()
    H.assert_quant_equal(bq, sc.quantize_w(H.bf16_bits(w), idx.numpy(), kn, ks, ko), n, (kn, ks, ko), what="c0 w")
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    _check_gemm(d, qx, qw, "c0")
    # the quantized product tracks the unquantized bf16 matmul (what main.py prints as MSE)
    full = x.float() @ w.float().T
    rel = (d.float().cpu() - full).norm() / full.norm()
    assert rel < 0.2, rel


# ------------------------------------------------------------------ the benchmark configurations at full size
@pytest.mark.parametrize("cfg", ["c2", "c3", "c4"])
def test_full_size_configs(abi, cfg):
    """At the sizes the bench runs: weights bit-exact against the scalar oracle; a sample of token rows
    (all of them for c2) against the oracle's GEMM; and two properties that need no oracle and cover every
    tile -- repeated runs are bit-identical, permuting the token rows permutes the output rows bit for bit (a
    row's arithmetic does not depend on where its tile sits), and doubling the activations (exact in bf16: codes unchanged, scale
    exponents + 1) doubles every output exactly."""
    m, n, k, kn, ks, ko = H.CONFIGS[cfg]
    _say(cfg, "full size", m, n, k)
    student = cfg == "c4"
    x = H.make_activations(m, k, 1234 + int(cfg[1]), student_t=student)
    w = H.make_weights(n, k, 2234 + int(cfg[1]))
    idx = H.absmax_sort_index(x)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    tiled = abi.weights_tileable(n, kn, ks, ko)
    bt = (abi.tile_weights(*bq[:3]) + bq[3:]) if tiled else bq
    d = abi.fused_linear(xd, idd, *bt, kn, ks, ko, w_tiled=tiled)
    torch.cuda.synchronize()
    H.assert_quant_equal(bq, sc.quantize_w(H.bf16_bits(w), idx.numpy(), kn, ks, ko), n, (kn, ks, ko), what=f"{cfg} w")

    # sampled token rows against the oracle
    rng = np.random.default_rng(7)
    rows = np.arange(m) if m <= 64 else np.sort(rng.choice(m, 48, replace=False))
    qx = mo.reorder_quantize_x(H.bf16_f32(x)[rows], idx.numpy(), kn, ks, ko)
    qw = mo.reorder_quantize_w(H.bf16_f32(w), idx.numpy(), kn, ks, ko)
    _check_gemm(d[torch.from_numpy(rows).to(DEV)], qx, qw, f"{cfg} sampled rows")
    aq = abi.reorder_quantize_x(xd, idd, kn, ks, ko)
    torch.cuda.synchronize()
    want = sc.quantize_x(H.bf16_bits(x)[rows], idx.numpy(), kn, ks, ko)
    for t, name in zip(aq[:3], ("qn", "qs", "qo")):
        np.testing.assert_array_equal(t.cpu().numpy()[rows], want[name], err_msg=f"{cfg} {name}")

    # the same launch again, twice, with other work in between: bit-identical (no race in the copy pipeline)
    for _ in range(2):
        abi.reorder_quantize_w(wd, idd, kn, ks, ko)
        again = abi.fused_linear(xd, idd, *bt, kn, ks, ko, w_tiled=tiled)
        torch.cuda.synchronize()
        assert torch.equal(again, d), f"{cfg}: two runs of the same problem differ"

    # token-row permutation
    perm = torch.from_numpy(rng.permutation(m)).to(DEV)
    d_perm = abi.fused_linear(xd[perm].contiguous(), idd, *bt, kn, ks, ko, w_tiled=tiled)
    torch.cuda.synchronize()
    assert torch.equal(d_perm, d[perm]), f"{cfg}: output rows do not follow a permutation of the token rows"

    # activations x 2
    d2 = abi.fused_linear((xd.float() * 2.0).to(torch.bfloat16), idd, *bt, kn, ks, ko, w_tiled=tiled)
    torch.cuda.synchronize()
    assert torch.equal(d2.float(), d.float() * 2.0), f"{cfg}: doubling the activations does not double the output"


# ------------------------------------------------------------------ torch extension surface
def test_extension_module_runs_the_reference_call_sequence(abi):
    import os
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "build"))
    import mixedgemm
    m, n, k = 114, 3584, 3584                      # the smoke script's shape
    kn, ks, ko = 2560, 3584 - 128 - 2560, 128
    x = H.make_activations(m, k, 77)
    w = H.make_weights(n, k, 78, std=1.0)
    idx = torch.arange(k, dtype=torch.int16)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    AN, AS, AO, SFAN, SFAS, SFAO = mixedgemm.reorder_quantize_x(xd, idd, kn, ks, ko, m, n)
    BN, BS, BO, SFBN, SFBS, SFBO = mixedgemm.reorder_quantize_w(wd, idd, kn, ks, ko, m, n)
    C = mixedgemm.matmul(AN, BN, AS, BS, AO, BO, SFAN, SFBN, SFAS, SFBS, SFAO, SFBO)
    assert C.shape == (m, n) and C.dtype == torch.bfloat16
    assert AN.shape == (m, kn // 2) and AS.shape == (m, ks // 4 * 3) and AO.shape == (m, ko)
    assert SFAN.numel() == (m // 128 + 1) * 128 * kn // 32 and SFBN.numel() == n * kn // 32
    H.assert_quant_equal((AN, AS, AO, SFAN, SFAS, SFAO), sc.quantize_x(H.bf16_bits(x), idx.numpy(), kn, ks, ko), m, (kn, ks, ko))
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    _check_gemm(C, qx, qw, "extension")
    with pytest.raises(RuntimeError):
        mixedgemm.reorder_quantize_x(xd, idd.to(torch.int32), kn, ks, ko, m, n)


@pytest.mark.parametrize("m,k", [(1, 32), (7, 96), (64, 4096), (129, 2080), (300, 14336), (4096, 4096), (33, 32736)])
def test_calibrate_reorder_index_matches_oracle(abi, m, k):
    """Per-channel absmax + stable ascending sort: identical index to the oracle, including the
    order of ties (coarse values make many) and channels that are entirely zero."""
    _say("calibrate", m, k)
    g = torch.Generator().manual_seed(m * 131 + k)
    if k <= 4096:
        x = (torch.randint(-6, 7, (m, k), generator=g).float() * 0.25).bfloat16()    # many ties
        x[:, ::17] = 0
    else:
        x = H.make_activations(m, k, m + k)
    idx = abi.calibrate_reorder_index(x.cuda())
    torch.cuda.synchronize()
    np.testing.assert_array_equal(idx.cpu().numpy(), mo.calibrate_reorder_index(H.bf16_bits(x)))


# ------------------------------------------------------------------ committed golden vectors
import glob as _glob
import os as _os

GOLDEN = sorted(_glob.glob(_os.path.join(_os.path.dirname(__file__), "golden", "path_*.npz")))


@pytest.mark.parametrize("path", GOLDEN, ids=[_os.path.basename(p) for p in GOLDEN])
def test_whole_path_matches_golden_vectors(abi, path):
    """Calibrate -> quantize both operands -> GEMM, on the inputs of a committed fixture."""
    _say("golden", _os.path.basename(path))
    g = np.load(path)
    kn, ks, ko = (int(v) for v in g["split"])
    x = torch.from_numpy(g["x_bits"].view(np.int16)).view(torch.bfloat16).to(DEV)
    w = torch.from_numpy(g["w_bits"].view(np.int16)).view(torch.bfloat16).to(DEV)
    idx = abi.calibrate_reorder_index(x)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(idx.cpu().numpy(), g["idx"])
    aq = abi.reorder_quantize_x(x, idx, kn, ks, ko)
    bq = abi.reorder_quantize_w(w, idx, kn, ks, ko)
    d = abi.matmul(aq[0], bq[0], aq[1], bq[1], aq[2], bq[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5])
    torch.cuda.synchronize()
    for tag, q, rows in (("x", aq, x.shape[0]), ("w", bq, w.shape[0])):
        for t, c in zip(q[:3], ("qn", "qs", "qo")):
            np.testing.assert_array_equal(t.cpu().numpy(), g[f"{tag}_{c}"], err_msg=f"{tag} {c}")
        for t, s, kseg in zip(q[3:], ("sfn", "sfs", "sfo"), (kn, ks, ko)):
            np.testing.assert_array_equal(H.gather_logical_scales(t, rows, kseg), g[f"{tag}_{s}"], err_msg=f"{tag} {s}")
    ref = g["d_f32"]
    err = np.abs(d.float().cpu().numpy() - mo.bf16_rne(ref))
    # 1 bf16 ulp for the final rounding + 2^-20 of sum |a||b| for the order of the fp32 accumulation
    assert np.all(err <= H.bf16_ulp(ref) + g["d_abs_f32"] * 2.0 ** -20), f"max err {err.max()}"


# ------------------------------------------------------------------ tile-major weights
def _tile_reference(w: np.ndarray) -> np.ndarray:
    """Tile-major order of one segment's weight codes [N, kseg/2] (N % 256 == 0, kseg % 32 == 0): whole
    128-wide stages as [feature tile][stage][block j][lane quad k][64 bytes], row = 256 * tile + j +
    16 * (2 * (k % 8) + k // 8); behind them what is left of every row, row-major."""
    n, cols = w.shape
    stages = cols // 64
    v = w[:, :stages * 64].reshape(n // 256, 256, stages, 64)
    k = np.arange(16)
    pr = 2 * (k % 8) + k // 8
    rows = (np.arange(16)[:, None] + 16 * pr[None, :])            # [j, k]
    out = v[:, rows, :, :]                                         # [tile, j, k, stage, 64]
    tiled = np.ascontiguousarray(out.transpose(0, 3, 1, 2, 4)).reshape(-1)
    return np.concatenate([tiled, np.ascontiguousarray(w[:, stages * 64:]).reshape(-1)]).reshape(n, cols)


@pytest.mark.parametrize("n,kseg", [(256, 128), (512, 384), (768, 2560), (256, 224), (512, 4928), (256, 160)])
def test_tile_weights_matches_the_layout_formula(abi, n, kseg):
    rng = np.random.default_rng(n + kseg)
    w = rng.integers(0, 256, (n, kseg // 2), dtype=np.uint8)
    z = torch.zeros((n, 64), dtype=torch.uint8, device=DEV)
    wd = torch.from_numpy(w).to(DEV)
    t = abi.tile_weights(wd, wd[:, :64].contiguous(), wd[:, :64].contiguous())
    torch.cuda.synchronize()
    np.testing.assert_array_equal(t[0].cpu().numpy(), _tile_reference(w))
    np.testing.assert_array_equal(t[1].cpu().numpy(), _tile_reference(w[:, :64]))
    del z


TILED_SHAPES = [
    # M, N, KN, KS, KO: the 256x256 kernel (plain and with compiled-in segment-boundary copies), ragged
    # token counts, and the skinny kernel with 1, 2, 4 and 8 token groups
    (256, 256, 128, 128, 128), (512, 512, 256, 384, 128), (256, 768, 2560, 1408, 128), (512, 256, 384, 512, 256),
    (300, 512, 2560, 1408, 128), (1000, 256, 384, 384, 384),
    (8, 512, 2560, 1408, 128), (20, 256, 128, 256, 128), (50, 768, 384, 128, 128), (130, 256, 2560, 896, 128),
    # plans without E3M2 and / or E4M3 activations
    (256, 256, 512, 0, 0), (300, 512, 384, 0, 128), (512, 256, 2560, 1536, 0), (40, 256, 1024, 0, 0),
    # segments that end 32, 64 or 96 elements past their last whole stage (kept row-major behind the tiled part)
    (256, 256, 448, 416, 224), (512, 512, 2240, 1248, 448), (300, 256, 160, 480, 352), (8, 256, 448, 416, 224),
    (40, 512, 2240, 1248, 448),
]


@pytest.mark.parametrize("m,n,kn,ks,ko", TILED_SHAPES)
def test_tiled_weights_give_the_same_result_bit_for_bit(abi, m, n, kn, ks, ko):
    """Tile-major weights change where a copy reads from, not what is multiplied or in which order."""
    _say("tiled", m, n, kn, ks, ko)
    k = kn + ks + ko
    x = H.make_activations(m, k, 31 + m + n, n_out=max(1, k // 32))
    w = H.make_weights(n, k, 33 + m + n)
    idx = H.absmax_sort_index(x)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    assert abi.weights_tileable(n, kn, ks, ko)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    bt = abi.tile_weights(*bq[:3])
    aq = abi.reorder_quantize_x(xd, idd, kn, ks, ko)
    d0 = abi.matmul(aq[0], bq[0], aq[1], bq[1], aq[2], bq[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5])
    d1 = abi.matmul(aq[0], bt[0], aq[1], bt[1], aq[2], bt[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5], w_tiled=True)
    d2 = abi.fused_linear(xd, idd, bt[0], bt[1], bt[2], bq[3], bq[4], bq[5], kn, ks, ko, w_tiled=True)
    tight = [t.clone() for t in aq]    # exact-size activation buffers
    d3 = abi.matmul(tight[0], bt[0], tight[1], bt[1], tight[2], bt[2], tight[3], bq[3], tight[4], bq[4], tight[5], bq[5],
                    w_tiled=True)
    torch.cuda.synchronize()
    assert torch.equal(d0, d1) and torch.equal(d0, d2)
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    _check_gemm(d1, qx, qw, "tiled")
    _check_gemm(d3, qx, qw, "tiled, exact-size buffers")


@pytest.mark.parametrize("m,m_part,n,kn,ks,ko", [
    # 272 whole tiles: 256 + 16 run as 32 half tiles; the first 4096 rows alone are 256 whole tiles, one round
    (4352, 4096, 4096, 384, 384, 128), (4352, 4096, 4096, 448, 416, 224), (4200, 4096, 4096, 384, 384, 384),
    # 144 whole tiles against 128 (at most half of the CUs: all of them as half tiles)
    (2304, 2048, 4096, 480, 448, 192),
])
def test_mixed_tile_heights_equal_the_plain_launch_bit_for_bit(abi, m, m_part, n, kn, ks, ko):
    """A launch that runs its last round (or all of its tiles) as 256 x 128 tiles adds the same products in the same
    order per output element as one that runs 256 x 256 tiles: the rows the two have in common are equal bit for
    bit.  The part call sees the first m_part token rows only (code rows and scale atoms are prefixes)."""
    _say("mixed tile heights", m, m_part, n, kn, ks, ko)
    k = kn + ks + ko
    x = H.make_activations(m, k, 71 + m + n, n_out=max(1, k // 32))
    w = H.make_weights(n, k, 73 + m + n)
    idx = H.absmax_sort_index(x)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    if abi.weights_tileable(n, kn, ks, ko):
        bq = abi.tile_weights(*bq[:3]) + bq[3:]
        tiled = True
    else:
        tiled = False
    aq = abi.reorder_quantize_x(xd, idd, kn, ks, ko)
    full = abi.matmul(aq[0], bq[0], aq[1], bq[1], aq[2], bq[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5], w_tiled=tiled)
    part_ops = [aq[0][:m_part].clone(), aq[1][:m_part].clone(), aq[2][:m_part].clone()]
    part_sf = [aq[3 + i][:abi.sf_bytes(m_part, kseg, abi.MG_OPERAND_A)].clone() for i, kseg in enumerate((kn, ks, ko))]
    part = abi.matmul(part_ops[0], bq[0], part_ops[1], bq[1], part_ops[2], bq[2], part_sf[0], bq[3], part_sf[1], bq[4],
                      part_sf[2], bq[5], w_tiled=tiled)
    torch.cuda.synchronize()
    assert torch.equal(full[:m_part], part)
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    _check_gemm(full, qx, qw, "mixed tile heights")


@pytest.mark.parametrize("m", [257, 258, 261, 263, 271, 272, 273, 384, 385, 511, 16, 129, 200])
@pytest.mark.parametrize("n,kn,ks,ko", [(2048, 2560, 1408, 128), (512, 448, 416, 224)])
def test_exact_size_activation_buffers_on_the_whole_tile_kernel(abi, m, n, kn, ks, ko):
    """Activation buffers with no room past row M: the lanes of the last tile that would read past the last row
    read that row again, and the result equals the padded-buffer one bit for bit.  Row counts around the lengths
    of the runs of rows a lane copies (2, 4, 8), the 16-row copy blocks and the second scale atom (128 rows)."""
    _say("exact-size", m, n, kn, ks, ko)
    k = kn + ks + ko
    x = H.make_activations(m, k, 71 + m, n_out=max(1, k // 32))
    w = H.make_weights(n, k, 72 + n)
    idx = H.absmax_sort_index(x)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    bt = abi.tile_weights(*bq[:3])
    aq = abi.reorder_quantize_x(xd, idd, kn, ks, ko)
    tight = [t.clone() for t in aq]
    assert all(t.untyped_storage().nbytes() == t.numel() for t in tight)
    args = lambda a, b: (a[0], b[0], a[1], b[1], a[2], b[2], a[3], bq[3], a[4], bq[4], a[5], bq[5])
    d_pad = abi.matmul(*args(aq, bq))
    d_tight = abi.matmul(*args(tight, bq))
    d_tight_t = abi.matmul(*args(tight, bt), w_tiled=True)
    torch.cuda.synchronize()
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    _check_gemm(d_tight, qx, qw, "exact-size buffers")
    assert torch.equal(d_tight, d_tight_t)
    assert torch.equal(d_pad, d_tight)


def _seeded_shapes(count, seed):
    """Shapes drawn across the dispatcher's cases: token counts on both sides of 256 and of whole tiles, feature
    counts with and without whole 256-feature tiles, segments of 0 or 32..1024 channels in steps of 32."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        m = int(rng.choice([rng.integers(1, 40), rng.integers(40, 256), rng.integers(256, 700)]))
        n = int(rng.choice([256 * rng.integers(1, 3), 16 * rng.integers(1, 40), rng.integers(1, 300)]))
        seg = lambda: int(rng.choice([0, 32 * rng.integers(1, 8), 128 * rng.integers(1, 8)]))
        kn, ks, ko = seg(), seg(), seg()
        if kn + ks + ko == 0:
            continue
        out.append((m, n, kn, ks, ko))
    return out


def _seeded_tile_shapes(count, seed):
    """Shapes the whole-tile kernel takes: ragged token counts, segments of whole stages or with 32, 64, 96 channels
    past them, with and without three stages before a boundary, plans without E3M2 and / or E4M3."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        m = int(rng.integers(1, 600))
        n = 256 * int(rng.integers(1, 3))
        kn = int(rng.choice([128 * rng.integers(1, 9), 128 + 32 * rng.integers(0, 30)]))
        ks = int(rng.choice([0, 128 * rng.integers(1, 7), 128 + 32 * rng.integers(0, 20)]))
        ko = int(rng.choice([0, 128 * rng.integers(1, 4), 128 + 32 * rng.integers(0, 8)]))
        out.append((m, n, kn, ks, ko))
    return out


@pytest.mark.parametrize("m,n,kn,ks,ko", _seeded_shapes(48, 20250) + _seeded_tile_shapes(40, 777))
def test_seeded_shape_sweep_against_the_oracle(abi, m, n, kn, ks, ko):
    """Whatever kernel the dispatcher picks, quantize + GEMM (padded and exact-size activation buffers, row-major
    and, where the shape allows it, tile-major weights) agree with the oracle and with each other."""
    _say("sweep", m, n, kn, ks, ko)
    k = kn + ks + ko
    x = H.make_activations(m, k, 7 + m + k, n_out=max(1, k // 32))
    w = H.make_weights(n, k, 9 + n + k)
    idx = H.random_index(k, m + n)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    aq = abi.reorder_quantize_x(xd, idd, kn, ks, ko)
    tight = [t.clone() for t in aq]
    args = lambda a, b: (a[0], b[0], a[1], b[1], a[2], b[2], a[3], bq[3], a[4], bq[4], a[5], bq[5])
    d_pad = abi.matmul(*args(aq, bq))
    d_tight = abi.matmul(*args(tight, bq))
    d_fused = abi.fused_linear(xd, idd, *bq, kn, ks, ko)
    torch.cuda.synchronize()
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    _check_gemm(d_pad, qx, qw, "padded buffers")
    _check_gemm(d_tight, qx, qw, "exact-size buffers")
    assert torch.equal(d_pad, d_fused)
    if abi.weights_tileable(n, kn, ks, ko):
        bt = abi.tile_weights(*bq[:3])
        d_t = abi.matmul(*args(tight, bt), w_tiled=True)
        torch.cuda.synchronize()
        _check_gemm(d_t, qx, qw, "tile-major weights")


def test_tiled_flag_is_refused_for_shapes_that_cannot_be_tiled(abi):
    from mixedgemm_amd.abi import MixedGemmError
    assert not abi.weights_tileable(256, 448, 416, 64) and not abi.weights_tileable(200, 128, 128, 128)
    m, n, kn, ks, ko = 16, 256, 448, 416, 64
    x = H.make_activations(m, kn + ks + ko, 3).to(DEV)
    idx = H.random_index(kn + ks + ko, 4).to(DEV)
    aq = abi.reorder_quantize_x(x, idx, kn, ks, ko)
    bq = abi.reorder_quantize_w(H.make_weights(n, kn + ks + ko, 5).to(DEV), idx, kn, ks, ko)
    with pytest.raises(MixedGemmError):
        abi.matmul(aq[0], bq[0], aq[1], bq[1], aq[2], bq[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5], w_tiled=True)


# ------------------------------------------------------------------ RMSNorm fused into the quantizer
@pytest.mark.parametrize("rows,kn,ks,ko,eps", [
    (7, 2560, 1408, 128, 1e-5), (130, 2560, 896, 128, 1e-6), (5, 128, 64, 64, 0.0),
    (9, 8960, 4928, 448, 1e-5),      # K = 14336: one lane per block, 448-lane workgroups
    (3, 11776, 6560, 608, 1e-5),     # K = 18944: 640-lane workgroups
    (1030, 256, 128, 128, 1e-5),     # more rows than resident workgroups: several rows per workgroup
    (5, 20480, 11264, 992, 1e-5),    # K = 32736, the largest: the kernel with a run-time workgroup size (1024 lanes)
    (300, 15360, 8448, 768, 1e-6),   # K = 24576 on the same kernel, two rows per workgroup for some
])
def test_rmsnorm_reorder_quantize_matches_oracle(abi, rows, kn, ks, ko, eps):
    k = kn + ks + ko
    _say("norm quant", rows, kn, ks, ko)
    x = H.make_activations(rows, k, 300 + rows, n_out=max(1, k // 32))
    g = torch.Generator().manual_seed(rows)
    gamma = (torch.randn(k, generator=g) * 0.3 + 1.0).to(torch.bfloat16)
    idx = H.random_index(k, 301 + rows)
    got = abi.rmsnorm_reorder_quantize_x(x.to(DEV), gamma.to(DEV), eps, idx.to(DEV), kn, ks, ko)
    torch.cuda.synchronize()
    y_bits = mo.rmsnorm_bf16(H.bf16_bits(x), H.bf16_bits(gamma), eps)
    want = sc.quantize_x(y_bits, idx.numpy(), kn, ks, ko)
    H.assert_quant_equal(got, want, rows, (kn, ks, ko), what=f"norm x {rows}x{k}")


@pytest.mark.parametrize("m,n,kn,ks,ko,eps", [
    (300, 512, 2560, 1408, 128, 1e-5),
    (40, 256, 15360, 8448, 768, 1e-5),    # K = 24576: the quantizer with a run-time workgroup size
])
def test_fused_norm_linear_equals_norm_then_linear(abi, m, n, kn, ks, ko, eps):
    k = kn + ks + ko
    x = H.make_activations(m, k, 61)
    w = H.make_weights(n, k, 62)
    g = torch.Generator().manual_seed(63)
    gamma = (torch.randn(k, generator=g) * 0.3 + 1.0).to(torch.bfloat16)
    y = torch.from_numpy(mo.rmsnorm_bf16(H.bf16_bits(x), H.bf16_bits(gamma), eps).view(np.int16)).view(torch.bfloat16)
    idx = H.absmax_sort_index(y)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    d1 = abi.fused_linear(xd, idd, *bq, kn, ks, ko, norm_weight=gamma.to(DEV), eps=eps)
    d2 = abi.fused_linear(y.to(DEV), idd, *bq, kn, ks, ko)
    torch.cuda.synchronize()
    assert torch.equal(d1, d2)
    qx, qw = _oracle_operands(y, w, idx, kn, ks, ko)
    _check_gemm(d1, qx, qw, "fused norm linear")


# ------------------------------------------------------------------ host-side argument checks and empty problems
def test_wrong_outputs_and_mismatched_operands_are_refused(abi):
    from mixedgemm_amd.abi import MixedGemmError
    m, n, kn, ks, ko = 8, 32, 128, 128, 128
    k = kn + ks + ko
    x = H.make_activations(m, k, 1).to(DEV)
    idx = H.random_index(k, 2).to(DEV)
    aq = abi.reorder_quantize_x(x, idx, kn, ks, ko)
    bq = abi.reorder_quantize_w(H.make_weights(n, k, 3).to(DEV), idx, kn, ks, ko)
    args = (aq[0], bq[0], aq[1], bq[1], aq[2], bq[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5])
    with pytest.raises(MixedGemmError):
        abi.matmul(*args, out=torch.empty((m, n + 1), dtype=torch.bfloat16, device=DEV))
    with pytest.raises(MixedGemmError):
        abi.matmul(*args, out=torch.empty((m, n), dtype=torch.float16, device=DEV))
    with pytest.raises(MixedGemmError):     # weights quantized with another split
        b2 = abi.reorder_quantize_w(H.make_weights(n, k, 3).to(DEV), idx, 256, 64, 64)
        abi.matmul(aq[0], b2[0], aq[1], b2[1], aq[2], b2[2], aq[3], b2[3], aq[4], b2[4], aq[5], b2[5])
    with pytest.raises(MixedGemmError):
        abi.reorder_quantize_x(x, idx, kn, ks, ko, out=aq[:5])
    with pytest.raises(MixedGemmError):
        abi.fused_linear(x, idx, *bq, kn, ks, ko, workspace=torch.empty(16, dtype=torch.uint8, device=DEV))
    with pytest.raises(MixedGemmError):
        abi.reorder_quantize_x(x, idx[:-1].contiguous(), kn, ks, ko)


def test_empty_problems(abi):
    kn, ks, ko = 128, 128, 128
    k = kn + ks + ko
    idx = H.random_index(k, 2).to(DEV)
    x0 = torch.empty((0, k), dtype=torch.bfloat16, device=DEV)
    aq = abi.reorder_quantize_x(x0, idx, kn, ks, ko)
    assert aq[0].shape == (0, kn // 2)
    bq = abi.reorder_quantize_w(H.make_weights(32, k, 3).to(DEV), idx, kn, ks, ko)
    d = abi.matmul(aq[0], bq[0], aq[1], bq[1], aq[2], bq[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5])
    assert d.shape == (0, 32)
    d = abi.fused_linear(x0, idx, *bq, kn, ks, ko)
    torch.cuda.synchronize()
    assert d.shape == (0, 32)

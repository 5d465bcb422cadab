"""Pins for the CPU oracle: every function of oracle/mx_oracle.py is checked
against something that is not a retyping of its own formula -- a library
routine (torch float8 casts), the independent scalar C derivation
(oracle/ref_scalar.c, which follows the reference's float formula with libm),
closed-form invariants, or brute force on tiny inputs."""
import itertools

import numpy as np
import pytest
import torch

from oracle import mx_oracle as mo
from oracle import scalar as sc


def all_positive_bf16():
    bits = np.arange(1, 0x7F80, dtype=np.uint32)            # denormals + normals, no inf/nan
    return (bits << 16).view(np.float32)


# ---------------------------------------------------------------- formats
def test_e2m1_grid_is_the_ocp_table():
    assert mo.format_grid("e2m1").tolist() == [0, 0.5, 1, 1.5, 2, 3, 4, 6]


def test_e3m2_grid_closed_form():
    g = mo.format_grid("e3m2")
    assert g.size == 32 and g[0] == 0 and g[1] == 0.0625 and g[3] == 0.1875
    assert g[4] == 0.25 and g[-1] == 28.0 and g[-2] == 24.0
    assert np.all(np.diff(g) > 0)


def test_e4m3_grid_matches_torch_decode():
    codes = torch.arange(0, 0x7F, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float().numpy()
    np.testing.assert_array_equal(mo.format_grid("e4m3")[:0x7F].astype(np.float32), ref)
    assert np.isnan(mo.format_grid("e4m3")[0x7F])


def _probe_values(fmt):
    g = mo.format_grid(fmt)
    g = g[~np.isnan(g)]
    mids = (g[:-1] + g[1:]) / 2
    eps = np.concatenate([mids * (1 + 2.0 ** -20), mids * (1 - 2.0 ** -20)])
    rnd = np.random.default_rng(0).uniform(0, g[-1] * 1.1, 4000)
    ints = np.arange(0, int(g[-1]) + 2, dtype=np.float64)
    return np.concatenate([g, mids, eps, rnd, ints]).astype(np.float32)


def test_e4m3_rounding_matches_torch_cast():
    v = _probe_values("e4m3")
    ref = torch.from_numpy(v).clamp(max=448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.testing.assert_array_equal(mo.rne_to_format(v, "e4m3"), ref)


@pytest.mark.parametrize("fmt", ["e2m1", "e3m2", "e4m3"])
def test_grid_search_rounding_matches_bit_manipulation(fmt):
    v = _probe_values(fmt)
    got = mo.rne_to_format(v, fmt)
    ref = np.array([sc.f32_to_exmy(x, fmt) for x in v], dtype=np.uint8)
    np.testing.assert_array_equal(got, ref)


def test_sign_of_zero_is_kept_by_converter():
    assert sc.f32_to_exmy(-0.0, "e2m1") == 0x8
    assert sc.f32_to_exmy(-0.0, "e3m2") == 0x20
    assert sc.f32_to_exmy(-0.0, "e4m3") == 0x80


def test_integer_luts_known_answers():
    assert mo.integer_lut("e2m1").tolist() == [0, 2, 4, 5, 6, 6, 7]
    assert mo.integer_lut("e3m2").tolist() == [
        0, 12, 16, 18, 20, 21, 22, 23, 24, 24, 25, 26, 26, 26, 27, 28, 28, 28, 28,
        29, 29, 29, 30, 30, 30, 30, 30, 31, 31]
    lut8 = mo.integer_lut("e4m3")
    # every integer up to 16 is exact in E4M3
    dec = mo.format_grid("e4m3")
    assert [dec[c] for c in lut8[:17]] == list(range(17))
    assert dec[lut8[448]] == 448 and dec[lut8[447]] == 448 and dec[lut8[17]] == 16
    # the bf16 hop (bf16 steps by 2 above 256) changes the direct RNE result at
    # exactly these integers
    direct = mo.rne_to_format(np.arange(449, dtype=np.float64), "e4m3")
    assert np.nonzero(direct != lut8)[0].tolist() == [273, 303, 337, 367, 401, 431]
    assert dec[lut8[273]] == 256 and dec[direct[273]] == 288


def test_integer_lut_matches_literal_c_chain():
    # C: roundf -> clamp -> bf16 -> bit-manipulation converter, through quant_block
    for fmt, maxv in (("e2m1", 6), ("e3m2", 28), ("e4m3", 448)):
        lut = mo.integer_lut(fmt)
        for v in range(maxv + 1):
            bf = mo.bf16_rne(np.float32(v))
            assert sc.f32_to_exmy(float(bf), fmt) == lut[v]


def test_bf16_rne_matches_torch():
    v = np.random.default_rng(1).standard_normal(20000).astype(np.float32) * 300
    v = np.concatenate([v, np.arange(0, 449, dtype=np.float32), [257.0, 259.0, 258.5]]).astype(np.float32)
    ref = torch.from_numpy(v).to(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(mo.bf16_rne(v), ref)


# ---------------------------------------------------------------- scale
@pytest.mark.parametrize("fmt", ["e2m1", "e3m2", "e4m3"])
def test_scale_exponent_closed_form_vs_float_formula_all_bf16(fmt):
    amax = all_positive_bf16()
    e = mo.scale_exponent(amax, fmt)
    maxv = mo.FORMATS[fmt][3]
    # invariant: e is the least exponent with amax <= MAX*2^e (where not clamped)
    a64 = amax.astype(np.float64)
    free = e > -127
    assert np.all(a64[free] <= maxv * 2.0 ** e[free])
    assert np.all(a64[free] > maxv * 2.0 ** (e[free] - 1.0))
    assert np.all(a64[~free] <= maxv * 2.0 ** -127)
    # the reference's formula ceil(log2(amax/MAX)) evaluated in float with libm
    lib = sc.lib()
    ref = np.array([lib.orc_scale_exponent(float(a), maxv) for a in amax], dtype=np.int32)
    np.testing.assert_array_equal(e, ref)


def test_scale_exponent_known_answers():
    f = np.float32
    assert mo.scale_exponent(f(0.0), "e2m1") == -1          # scale 0.5
    assert mo.scale_exponent(f(6.0), "e2m1") == 0
    assert mo.scale_exponent(f(6.03125), "e2m1") == 1
    assert mo.scale_exponent(f(3.0), "e2m1") == -1
    assert mo.scale_exponent(f(1.0), "e2m1") == -2          # 1 <= 6/4, > 6/8
    assert mo.scale_exponent(f(28.0), "e3m2") == 0
    assert mo.scale_exponent(f(30.0), "e3m2") == 1
    assert mo.scale_exponent(f(448.0), "e4m3") == 0
    assert mo.scale_exponent(f(1.0), "e4m3") == -8          # 448/256 = 1.75 >= 1 > 0.875


def test_e8m0_byte_matches_torch_cast():
    e = np.arange(-126, 127)
    ref = torch.from_numpy(np.ldexp(np.float32(1), e)).to(torch.float8_e8m0fnu).view(torch.uint8).numpy()
    np.testing.assert_array_equal((e + 127).astype(np.uint8), ref)
    x = np.zeros((1, 1, 32), np.float32)
    codes, e8 = mo.quantize_blocks(x, "e2m1")
    assert e8.item() == 126 and not codes.any()


# ---------------------------------------------------------------- packing
def test_pack_fp4_hand_vector_and_round_trip():
    assert mo.pack_fp4(np.array([0x1, 0xA, 0xF, 0x0])).tolist() == [0xA1, 0x0F]
    c = np.random.default_rng(2).integers(0, 16, (5, 64), dtype=np.uint8)
    np.testing.assert_array_equal(mo.unpack_fp4(mo.pack_fp4(c)), c)


def test_pack_fp6_hand_vector_and_round_trip():
    # one-hot elements land at bits [6i, 6i+6) of the little-endian 24-bit word
    for i in range(4):
        c = np.zeros(4, np.uint8)
        c[i] = 0x3F
        b = mo.pack_fp6(c)
        word = int(b[0]) | int(b[1]) << 8 | int(b[2]) << 16
        assert word == 0x3F << (6 * i)
    assert mo.pack_fp6(np.array([0x21, 0x12, 0x3C, 0x07])).tolist() == [
        0x21 | (0x12 & 3) << 6, (0x12 >> 2) | (0x3C & 0xF) << 4, (0x3C >> 4) | 0x07 << 2]
    c = np.random.default_rng(3).integers(0, 64, (5, 64), dtype=np.uint8)
    np.testing.assert_array_equal(mo.unpack_fp6(mo.pack_fp6(c)), c)


# ---------------------------------------------------------------- scale layout
def test_sf_offset_hand_values():
    k = 2560                                                 # 20 K-atoms
    assert mo.sf_offset(0, 0, k) == 0
    assert mo.sf_offset(1, 0, k) == 16
    assert mo.sf_offset(31, 0, k) == 496
    assert mo.sf_offset(32, 0, k) == 4
    assert mo.sf_offset(127, 3, k) == 31 * 16 + 3 * 4 + 3 == 511
    assert mo.sf_offset(0, 4, k) == 512
    assert mo.sf_offset(128, 0, k) == 20 * 512
    assert mo.sf_offset(129, 5, k) == 21 * 512 + 16 + 1


@pytest.mark.parametrize("rows,kseg", [(128, 128), (130, 2560), (114, 896), (300, 1408), (8, 4928), (257, 448)])
def test_sf_offset_invariants(rows, kseg):
    nb = kseg // 32
    r, kb = np.meshgrid(np.arange(rows), np.arange(nb), indexing="ij")
    off = mo.sf_offset(r, kb, kseg)
    assert np.unique(off).size == off.size                                   # injective
    span = ((rows + 127) // 128) * ((kseg + 127) // 128) * 512
    assert off.max() < span <= mo.sf_bytes(rows, kseg, "a")
    assert span <= mo.sf_bytes(rows, kseg, "b")
    full = nb // 4 * 4
    o4 = off[:, :full].reshape(rows, -1, 4)
    assert np.all(o4[..., 0] % 4 == 0) and np.all(np.diff(o4, axis=-1) == 1)  # one aligned dword per 4 blocks
    # round trip through the buffer
    e8 = np.random.default_rng(4).integers(0, 255, (rows, nb), dtype=np.uint8)
    np.testing.assert_array_equal(mo.sf_gather(mo.sf_scatter(e8, kseg, "a"), rows, kseg), e8)


def test_sf_sizes_match_reference_allocation_when_aligned():
    # (M/128+1)*128*K/32 for activations, N*K/32 for weights
    assert mo.sf_bytes(114, 2560, "a") == 128 * 80
    assert mo.sf_bytes(4096, 1408, "a") == 33 * 128 * 44
    assert mo.sf_bytes(14336, 2560, "b") == 14336 * 80


# ---------------------------------------------------------------- quantizer
def _rand_bf16(rng, shape, scale=1.0):
    x = torch.from_numpy(rng.standard_normal(shape).astype(np.float32) * scale).to(torch.bfloat16)
    return x.float().numpy(), x.view(torch.int16).numpy().view(np.uint16)


def _adversarial_rows(k):
    """Rows of blocks built to hit the corners: zeros, -0.0, ties of roundf,
    ties of the element rounding, amax exactly MAX*2^e, denormals, huge values."""
    rows = []
    base = np.zeros(k, np.float32)
    rows.append(base.copy())
    r = base.copy(); r[:] = -0.0; rows.append(r)
    r = base.copy(); r[::32] = 6.0; r[1::32] = -0.25; r[2::32] = 2.5; r[3::32] = -4.5; r[4::32] = 5.0; r[5::32] = 0.5; rows.append(r)
    r = base.copy(); r[::32] = 28.0; r[1::32] = 9.0; r[2::32] = -13.0; r[3::32] = 26.0; r[4::32] = 10.5; r[5::32] = -0.4375; rows.append(r)
    r = base.copy(); r[::32] = 448.0; r[1::32] = 273.0; r[2::32] = -431.0; r[3::32] = 17.0; r[4::32] = 272.5; rows.append(r)
    r = base.copy(); r[::32] = 6.0 * 2.0 ** -20; r[1::32] = -5.0 * 2.0 ** -20; rows.append(r)
    r = base.copy(); r[::32] = 3.0e38; r[1::32] = -1.0e38; rows.append(r)
    r = base.copy(); r[::32] = 2.0 ** -120; r[1::32] = -(2.0 ** -121); rows.append(r)
    r = base.copy(); r[::32] = 6.03125; r[7::32] = 3.0; rows.append(r)
    x = torch.from_numpy(np.stack(rows)).to(torch.bfloat16)
    return x.float().numpy(), x.view(torch.int16).numpy().view(np.uint16)


SPLITS = [(4096, 2560, 1408, 128), (3584, 2560, 896, 128), (5120, 3072, 1920, 128),
          (14336, 8960, 4928, 448), (18944, 12288, 6400, 256), (12288, 7680, 4224, 384),
          (13824, 8704, 4736, 384), (256, 64, 96, 96), (128, 128, 0, 0), (96, 0, 64, 32)]


@pytest.mark.parametrize("k,kn,ks,ko", SPLITS)
def test_numpy_oracle_matches_scalar_c_oracle(k, kn, ks, ko):
    rng = np.random.default_rng(k)
    xf, xb = _rand_bf16(rng, (5, k))
    xf[:, ::97] *= 30
    xb = torch.from_numpy(xf).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    xf = torch.from_numpy(xf).to(torch.bfloat16).float().numpy()
    af, ab = _adversarial_rows(k)
    xf, xb = np.concatenate([xf, af]), np.concatenate([xb, ab])
    idx = rng.permutation(k).astype(np.int16)
    for fn_np, fn_c in ((mo.reorder_quantize_x, sc.quantize_x), (mo.reorder_quantize_w, sc.quantize_w)):
        a, b = fn_np(xf, idx, kn, ks, ko), fn_c(xb, idx, kn, ks, ko)
        for name in ("qn", "qs", "qo", "sfn", "sfs", "sfo"):
            np.testing.assert_array_equal(a[name], b[name], err_msg=name)


def test_identity_index_is_plain_blockwise_quantization():
    rng = np.random.default_rng(7)
    xf, _ = _rand_bf16(rng, (3, 256))
    q = mo.reorder_quantize_x(xf, np.arange(256), 128, 64, 64)
    codes, e8 = mo.quantize_blocks(xf[:, :128].reshape(3, 4, 32), "e2m1")
    np.testing.assert_array_equal(q["codes_n"], codes.reshape(3, 128))
    np.testing.assert_array_equal(q["e8m0_n"], e8)


def test_gather_direction_and_within_block_permutation():
    rng = np.random.default_rng(8)
    xf, _ = _rand_bf16(rng, (2, 128))
    idx = rng.permutation(128)
    q = mo.reorder_quantize_x(xf, idx, 128, 0, 0)
    q_id = mo.reorder_quantize_x(xf[:, idx], np.arange(128), 128, 0, 0)     # out[:, j] = in[:, idx[j]]
    np.testing.assert_array_equal(q["qn"], q_id["qn"])
    # permuting inside each 32-block leaves every scale unchanged
    idx2 = idx.reshape(4, 32)[:, rng.permutation(32)].reshape(-1)
    np.testing.assert_array_equal(mo.reorder_quantize_x(xf, idx2, 128, 0, 0)["e8m0_n"], q["e8m0_n"])


def test_block_max_lands_in_upper_half_and_clamp_never_fires():
    rng = np.random.default_rng(9)
    xf, _ = _rand_bf16(rng, (16, 4096), 3.0)
    for fmt in ("e2m1", "e3m2", "e4m3"):
        maxv = mo.FORMATS[fmt][3]
        blocks = xf.reshape(16, 128, 32)
        _, e8 = mo.quantize_blocks(blocks, fmt)
        scaled = np.abs(blocks).max(-1) / np.ldexp(1.0, e8.astype(int) - 127)
        assert np.all(scaled <= maxv) and np.all(scaled > maxv / 2)


def test_dequantized_error_is_bounded_by_half_a_step():
    # |x/scale - decode(code)| <= 0.5 (integer rounding) + half the widest element gap
    rng = np.random.default_rng(10)
    xf, _ = _rand_bf16(rng, (8, 512))
    for fmt, gap in (("e2m1", 2.0), ("e3m2", 4.0), ("e4m3", 32.0)):
        blocks = xf.reshape(8, 16, 32)
        codes, e8 = mo.quantize_blocks(blocks, fmt)
        scale = np.ldexp(1.0, e8.astype(int) - 127)[..., None]
        err = np.abs(blocks / scale - mo.decode_codes(codes, fmt))
        assert err.max() <= 0.5 + gap / 2 + 1.0      # +1: bf16 hop above 256


# ---------------------------------------------------------------- GEMM
def test_mixed_matmul_brute_force_tiny():
    rng = np.random.default_rng(11)
    m, n, kn, ks, ko = 3, 4, 64, 32, 32
    k = kn + ks + ko
    xf, _ = _rand_bf16(rng, (m, k), 2.0)
    wf, _ = _rand_bf16(rng, (n, k), 0.05)
    idx = rng.permutation(k)
    qx, qw = mo.reorder_quantize_x(xf, idx, kn, ks, ko), mo.reorder_quantize_w(wf, idx, kn, ks, ko)
    grids = {f: mo.format_grid(f) for f in mo.FORMATS}

    def val(code, fmt):
        bits = mo.BITS[fmt]
        mag = grids[fmt][code & ((1 << (bits - 1)) - 1)]
        return -mag if code >> (bits - 1) else mag

    want = np.zeros((m, n))
    for i, j in itertools.product(range(m), range(n)):
        for name, fmt in (("n", "e2m1"), ("s", "e3m2"), ("o", "e4m3")):
            ca, cb = qx["codes_" + name], qw["codes_" + name]
            for kk in range(ca.shape[1]):
                sa = 2.0 ** (int(qx["e8m0_" + name][i, kk // 32]) - 127)
                sb = 2.0 ** (int(qw["e8m0_" + name][j, kk // 32]) - 127)
                want[i, j] += val(int(ca[i, kk]), fmt) * sa * val(int(cb[j, kk]), "e2m1") * sb
    np.testing.assert_allclose(mo.mixed_matmul(qx, qw), want.astype(np.float32), rtol=1e-6)
    # quantized product approximates the unquantized one
    assert np.abs(want - xf.astype(np.float64) @ wf.astype(np.float64).T).max() < 0.25 * np.abs(want).max() + 0.5


def test_chain_mode_rounds_three_times():
    rng = np.random.default_rng(12)
    xf, _ = _rand_bf16(rng, (4, 128), 2.0)
    wf, _ = _rand_bf16(rng, (8, 128), 0.5)
    idx = np.arange(128)
    qx, qw = mo.reorder_quantize_x(xf, idx, 64, 32, 32), mo.reorder_quantize_w(wf, idx, 64, 32, 32)
    full = mo.mixed_matmul(qx, qw)
    chained = mo.mixed_matmul(qx, qw, chain_bf16=True)
    np.testing.assert_array_equal(chained, mo.bf16_rne(chained))
    np.testing.assert_allclose(chained, full, rtol=3 * 2.0 ** -8, atol=1e-3)


# ---------------------------------------------------------------- calibration (reorder index)
def test_calibrate_index_matches_torch_sort_of_absmax():
    """The reference's recipe run literally on the CPU (torch.max(torch.abs(X), dim=0) ->
    torch.sort ascending -> int16, main.py:31-33), on data without ties where its result is
    unique, and with stable=True on data full of ties."""
    from tests import helpers as H
    g = torch.Generator().manual_seed(11)
    # 256 distinct bf16 magnitudes (consecutive bit patterns from 1.0 up), one per channel, as the
    # channel maxima; the other rows stay below them
    peak = (torch.arange(256, dtype=torch.int32) + 0x3F80).to(torch.int16).view(torch.bfloat16)[torch.randperm(256, generator=g)]
    x = (torch.rand(37, 256, generator=g) * 0.9 * peak.float()).bfloat16()
    x[11] = peak * (torch.randint(0, 2, (256,), generator=g) * 2 - 1).bfloat16()
    absmax = torch.max(torch.abs(x.float()), dim=0).values
    assert absmax.unique().numel() == absmax.numel()
    ref = torch.sort(absmax, descending=False).indices.to(torch.int16).numpy()
    np.testing.assert_array_equal(mo.calibrate_reorder_index(H.bf16_bits(x)), ref)
    # ties: few distinct magnitudes, negative zeros, a zero channel
    t = (torch.randint(-3, 4, (19, 128), generator=g).float() * 0.5).bfloat16()
    t[:, 5] = 0.0
    t[3, 7] = -0.0
    ref = torch.sort(torch.max(torch.abs(t.float()), dim=0).values, descending=False, stable=True).indices.to(torch.int16).numpy()
    np.testing.assert_array_equal(mo.calibrate_reorder_index(H.bf16_bits(t)), ref)


def test_calibrate_index_is_a_permutation_sorted_by_absmax():
    from tests import helpers as H
    x = H.make_activations(64, 4096, 5)
    idx = mo.calibrate_reorder_index(H.bf16_bits(x)).astype(np.int64)
    assert sorted(idx.tolist()) == list(range(4096))
    am = x.float().abs().max(dim=0).values.numpy()
    assert np.all(np.diff(am[idx]) >= 0)


# ------------------------------------------------------------------ RMSNorm in front of the quantizer
def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _from_bits(b):
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.bfloat16)


def test_rmsnorm_closed_forms():
    """Cases whose answer is known without the formula: a constant row normalises to +-1, so y is the
    weight itself (a sum in place of the mean, a missing square root or a dropped weight all fail this);
    scaling a row by a power of two changes nothing when eps = 0; a zero row stays zero with eps > 0."""
    g = torch.Generator().manual_seed(3)
    k = 256
    gamma = (torch.randn(k, generator=g) * 0.5 + 1.0).to(torch.bfloat16)
    x = torch.full((3, k), 1.5, dtype=torch.bfloat16)
    x[1] = -0.375
    x[2, ::2] = -1.5                                   # |x| constant, signs alternate
    y = _from_bits(mo.rmsnorm_bf16(_bits(x), _bits(gamma), 0.0)).float()
    np.testing.assert_array_equal(y[0].numpy(), gamma.float().numpy())
    np.testing.assert_array_equal(y[1].numpy(), -gamma.float().numpy())
    sign = torch.ones(k); sign[::2] = -1
    np.testing.assert_array_equal(y[2].numpy(), (gamma.float() * sign).numpy())
    xr = torch.randn(4, k, generator=g).to(torch.bfloat16)
    a = mo.rmsnorm_bf16(_bits(xr), _bits(gamma), 0.0)
    b = mo.rmsnorm_bf16(_bits((xr.float() * 64.0).to(torch.bfloat16)), _bits(gamma), 0.0)
    np.testing.assert_array_equal(a, b)
    z = mo.rmsnorm_bf16(_bits(torch.zeros(1, k, dtype=torch.bfloat16)), _bits(gamma), 1e-6)
    assert not (z & 0x7FFF).any()


def test_rmsnorm_agrees_with_the_usual_fp32_implementation():
    """torch, written the way transformer code writes it.  Its float32 mean and rsqrt may differ from the
    pinned float64 ones in the last bit, which can move a bf16 rounding: at most a few values per
    thousand may differ, each by one bf16 step."""
    g = torch.Generator().manual_seed(4)
    m, k, eps = 16, 4096, 1e-5
    x = (torch.randn(m, k, generator=g) * 3.0).to(torch.bfloat16)
    gamma = (torch.randn(k, generator=g) * 0.2 + 1.0).to(torch.bfloat16)
    h = x.float()
    var = h.pow(2).mean(-1, keepdim=True)
    ref = gamma * (h * torch.rsqrt(var + eps)).to(torch.bfloat16)
    got = _from_bits(mo.rmsnorm_bf16(_bits(x), _bits(gamma), eps))
    diff = (got.view(torch.int16).int() - ref.view(torch.int16).int()).abs()
    assert int(diff.max()) <= 1
    assert float((diff != 0).float().mean()) < 5e-3

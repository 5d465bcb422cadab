"""Host-side checks that need no GPU: the C-ABI library loads, exports every
symbol the header declares, and its host logic (sizes, offsets, validation that
happens before any launch) agrees with the oracle."""
import ctypes
import os
import re

import numpy as np
import pytest

from oracle import mx_oracle as mo

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mixedgemm_abi.h")


@pytest.fixture(scope="module")
def abi():
    from mixedgemm_amd import abi as a
    if not os.path.exists(a.LIB_PATH):
        from mixedgemm_amd import build
        build.build_hip_library()
    return a


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mg_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(abi):
    lib = ctypes.CDLL(abi.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 9
    for name in names:
        assert hasattr(lib, name), name
    assert set(names) == set(abi.SYMBOLS)


@pytest.mark.parametrize("rows,kseg", [(114, 2560), (4096, 1408), (8, 128), (2048, 4928), (2048, 448), (1, 32), (0, 128)])
def test_sf_bytes_and_offsets_match_oracle(abi, rows, kseg):
    assert abi.sf_bytes(rows, kseg, abi.MG_OPERAND_A) == mo.sf_bytes(rows, kseg, "a")
    assert abi.sf_bytes(rows, kseg, abi.MG_OPERAND_B) == mo.sf_bytes(rows, kseg, "b")
    rng = np.random.default_rng(rows + kseg)
    for _ in range(50):
        r, kb = int(rng.integers(0, max(rows, 1))), int(rng.integers(0, kseg // 32))
        assert abi.sf_offset(r, kb, kseg) == int(mo.sf_offset(r, kb, kseg))


def test_validation_rejects_bad_shapes_before_any_launch(abi):
    lib = abi.lib()
    null = ctypes.c_void_p(0)
    args = [null] * 6
    # a segment that is not a multiple of 32
    assert lib.mg_reorder_quantize_x(null, null, 4, 4096, 2560, 1400, 136, *args, null) == 10001
    # K != KN + KS + KO
    assert lib.mg_reorder_quantize_w(null, null, 4, 4000, 2560, 1408, 128, *args, null) == 10001
    # K beyond the int16 index range
    assert lib.mg_reorder_quantize_x(null, null, 4, 32768, 32768, 0, 0, *args, null) == 10004
    # null pointers with a non-empty problem
    assert lib.mg_reorder_quantize_x(null, null, 4, 4096, 2560, 1408, 128, *args, null) == 10002
    assert lib.mg_mixed_gemm(*([null] * 12), 4, 8, 128, 0, 0, null, null) == 10002
    # empty problems succeed without touching the device
    assert lib.mg_reorder_quantize_x(null, null, 0, 4096, 2560, 1408, 128, *args, null) == 0
    assert lib.mg_mixed_gemm(*([null] * 12), 0, 8, 128, 0, 0, null, null) == 0
    assert "multiples of 32" in abi.status_string(10001)


def test_validation_of_the_newer_entry_points(abi):
    lib = abi.lib()
    null = ctypes.c_void_p(0)
    twelve = [null] * 12
    assert lib.mg_padded_rows(0) == 0 and lib.mg_padded_rows(1) == 256 and lib.mg_padded_rows(256) == 256
    assert lib.mg_padded_rows(4000) == 4096
    assert lib.mg_weights_tileable(14336, 2560, 1408, 128) == 1
    assert lib.mg_weights_tileable(4096, 8960, 4928, 448) == 1      # 32-granular segments are fine
    assert lib.mg_weights_tileable(4096, 2560, 1408, 64) == 0       # a segment narrower than one stage
    assert lib.mg_weights_tileable(1000, 2560, 1408, 128) == 0      # N not a multiple of 256
    assert lib.mg_weights_tileable(256, 256, 0, 128) == 1           # an empty segment: whole stages in the others
    assert lib.mg_weights_tileable(256, 0, 384, 0) == 1 and lib.mg_weights_tileable(512, 0, 0, 128) == 1
    assert lib.mg_weights_tileable(256, 416, 0, 160) == 0           # an empty segment next to segments that are not whole stages
    # plans without one or two of the activation formats: whole 128-wide stages
    assert lib.mg_weights_tileable(256, 4096, 0, 0) == 1 and lib.mg_weights_tileable(256, 128, 0, 0) == 1
    assert lib.mg_weights_tileable(256, 3968, 0, 128) == 1 and lib.mg_weights_tileable(256, 2560, 1536, 0) == 1
    assert lib.mg_weights_tileable(256, 0, 3968, 128) == 1 and lib.mg_weights_tileable(256, 4064, 0, 32) == 0
    assert lib.mg_weights_tileable(256, -128, 0, 0) == 0 and lib.mg_weights_tileable(256, 512, -128, 0) == 0
    # a_rows below M, unknown flag bits, tile-major flag on a shape that cannot be tiled
    assert lib.mg_mixed_gemm_ex(*twelve, 8, 4, 256, 128, 128, 128, 0, null, null) == 10001
    assert lib.mg_mixed_gemm_ex(*twelve, 8, 8, 256, 128, 128, 128, 2, null, null) == 10001
    assert lib.mg_mixed_gemm_ex(*twelve, 8, 8, 256, 448, 416, 64, 1, null, null) == 10004
    # tiling: N and the segment width must be whole tiles / stages; in place is refused
    one = ctypes.c_void_p(256)
    assert lib.mg_tile_weights(one, ctypes.c_void_p(512), 200, 128, null) == 10001
    assert lib.mg_tile_weights(one, ctypes.c_void_p(512), 256, 100, null) == 10001
    assert lib.mg_tile_weights(one, one, 256, 128, null) == 10002
    assert lib.mg_tile_weights(null, null, 0, 128, null) == 0
    # the normalising quantizer needs a weight vector and eps >= 0
    six = [null] * 6
    assert lib.mg_rmsnorm_reorder_quantize_x(null, null, 1e-5, null, 4, 4096, 2560, 1408, 128, *six, null) == 10002
    assert lib.mg_rmsnorm_reorder_quantize_x(null, one, -1.0, null, 4, 4096, 2560, 1408, 128, *six, null) == 10001
    # calibration
    assert lib.mg_calibrate_reorder_index(null, 4, 100, null, null, 0, null) == 10001
    assert lib.mg_calibrate_reorder_index(null, 4, 32768, null, null, 0, null) == 10004
    assert lib.mg_calibrate_workspace_bytes(4096) >= 4096 * 4


def test_fused_workspace_size(abi):
    kn, ks, ko = 2560, 1408, 128
    for m in (4096, 300, 8):      # sized for whole 256-row tiles
        r = (m + 255) // 256 * 256
        need = abi.fused_workspace_bytes(m, kn, ks, ko)
        parts = [r * kn // 2, r * ks * 3 // 4, r * ko] + [mo.sf_bytes(r, k, "a") for k in (kn, ks, ko)]
        assert need == sum((p + 255) // 256 * 256 for p in parts)


def test_extension_module_surface():
    """The torch extension keeps the reference's operator names and keywords."""
    import sys
    ext = os.path.join(ROOT, "build", "mixedgemm.so")
    if not os.path.exists(ext):
        from mixedgemm_amd import build
        build.build_all()
    sys.path.insert(0, os.path.join(ROOT, "build"))
    import torch  # noqa: F401  (the extension links against libtorch)
    import mixedgemm
    assert mixedgemm.test_function() == "Hello from test_function!"
    for name in ("matmul", "reorder_quantize_x", "reorder_quantize_w"):
        assert callable(getattr(mixedgemm, name))
    doc = mixedgemm.reorder_quantize_x.__doc__
    for kw in ("X", "reorder_index", "KN", "KS", "KO", "seqlen", "outfeatures"):
        assert kw in doc
    doc = mixedgemm.matmul.__doc__
    for kw in ("AN", "BN", "AS", "BS", "AO", "BO", "SFAN", "SFBN", "SFAS", "SFBS", "SFAO", "SFBO"):
        assert kw in doc
    # invalid K: same exception type and message as the reference boundary
    x = torch.zeros(2, 100, dtype=torch.bfloat16)
    idx = torch.arange(100, dtype=torch.int16)
    with pytest.raises(RuntimeError, match="Value error in run_reorder_bf16_mixed"):
        mixedgemm.reorder_quantize_x(x, idx, 50, 30, 20, 2, 2)
    with pytest.raises(RuntimeError, match="Value error in run_reorder_bf16_fp4"):
        mixedgemm.reorder_quantize_w(x, idx, 50, 30, 20, 2, 2)


# ------------------------------------------------------------------ reorder index range, host side
def test_check_reorder_index_host(abi):
    import torch
    k = 256
    good = torch.randperm(k).to(torch.int16)
    abi.check_reorder_index(good)
    assert abi.lib().mg_check_reorder_index_host(ctypes.c_void_p(good.data_ptr()), k) == 0
    for pos, val in ((0, -1), (17, k), (255, 32767), (3, -32768)):
        bad = good.clone()
        bad[pos] = val
        assert abi.lib().mg_check_reorder_index_host(ctypes.c_void_p(bad.data_ptr()), k) == 10003
        with pytest.raises(abi.MixedGemmError, match="out of range"):
            abi.check_reorder_index(bad)
    with pytest.raises(abi.MixedGemmError):
        abi.check_reorder_index(good, k + 32)
    with pytest.raises(abi.MixedGemmError):
        abi.check_reorder_index(good.to(torch.int32))
    # repeats are a legal gather
    abi.check_reorder_index(torch.zeros(k, dtype=torch.int16))
    assert abi.lib().mg_check_reorder_index_host(ctypes.c_void_p(0), 0) == 0
    assert abi.lib().mg_check_reorder_index_host(ctypes.c_void_p(0), 32) == 10002
    assert "out of range" in abi.status_string(10003)


# ------------------------------------------------------------------ operand checks of the Python binding
class _NoLaunch:
    """Stands in for the loaded library: size queries go through, any compute entry point fails the test."""

    def __init__(self, real):
        self._real = real

    def __getattr__(self, name):
        if name in ("mg_sf_bytes", "mg_sf_offset", "mg_fused_workspace_bytes", "mg_padded_rows", "mg_status_string",
                    "mg_weights_tileable", "mg_calibrate_workspace_bytes", "mg_check_reorder_index_host"):
            return getattr(self._real, name)
        raise AssertionError(f"{name} reached with operands that should have been refused")


@pytest.fixture
def no_launch(abi, monkeypatch):
    """The binding with its GPU requirement lifted (CPU tensors pass the device check) and every launch
    turned into a test failure: what is left is the validation that runs before a launch."""
    import torch
    real = abi.lib()
    fake = _NoLaunch(real)
    monkeypatch.setattr(abi, "lib", lambda: fake)

    def require(t, dtype, name):
        if t.dtype != dtype:
            raise abi.MixedGemmError(f"{name}: expected {dtype}, got {t.dtype}")
        if not t.is_contiguous():
            raise abi.MixedGemmError(f"{name}: expected a contiguous tensor")

    monkeypatch.setattr(abi, "_require", require)
    monkeypatch.setattr(abi, "_stream", lambda t: ctypes.c_void_p(0))
    return abi


def _weights(abi, n, kn, ks, ko):
    import torch
    u8 = dict(dtype=torch.uint8)
    return [torch.zeros((n, kn // 2), **u8), torch.zeros((n, ks // 2), **u8), torch.zeros((n, ko // 2), **u8),
            torch.zeros(abi.sf_bytes(n, kn, abi.MG_OPERAND_B), **u8), torch.zeros(abi.sf_bytes(n, ks, abi.MG_OPERAND_B), **u8),
            torch.zeros(abi.sf_bytes(n, ko, abi.MG_OPERAND_B), **u8)]


def test_fused_linear_refuses_bad_weights_before_any_launch(no_launch):
    import torch
    abi = no_launch
    m, n, kn, ks, ko = 8, 64, 128, 64, 32
    k = kn + ks + ko
    x = torch.zeros((m, k), dtype=torch.bfloat16)
    idx = torch.arange(k, dtype=torch.int16)
    good = _weights(abi, n, kn, ks, ko)
    # a well-formed call gets as far as the launch
    with pytest.raises(AssertionError, match="mg_fused_norm_linear reached"):
        abi.fused_linear(x, idx, *good, kn, ks, ko)
    cases = {
        "wrong dtype": (0, good[0].to(torch.int8)),
        "too few rows in a segment": (1, good[1][:-1]),
        "wrong row width": (2, torch.zeros((n, ko // 2 + 16), dtype=torch.uint8)),
        "not contiguous": (0, torch.zeros((n, kn), dtype=torch.uint8)[:, ::2]),
        "1-D codes": (0, good[0].reshape(-1)),
        "short scale buffer": (3, good[3][:-1]),
        "short scale buffer (last segment)": (5, good[5][:1]),
        "float scales": (4, good[4].float()),
    }
    for what, (pos, t) in cases.items():
        ops = list(good)
        ops[pos] = t
        with pytest.raises(abi.MixedGemmError):
            abi.fused_linear(x, idx, *ops, kn, ks, ko)
        with pytest.raises(abi.MixedGemmError):
            abi.fused_linear_static(x, idx, *ops, kn, ks, ko, out=torch.zeros((m, n), dtype=torch.bfloat16))
    # the activations and the index
    with pytest.raises(abi.MixedGemmError):
        abi.fused_linear(x[:, :-32].contiguous(), idx, *good, kn, ks, ko)
    with pytest.raises(abi.MixedGemmError):
        abi.fused_linear(x, idx[:-1], *good, kn, ks, ko)
    with pytest.raises(abi.MixedGemmError):
        abi.fused_linear(x, idx, *good, kn, ks + 16, ko - 16)
    with pytest.raises(abi.MixedGemmError):
        abi.fused_linear(x, idx, *good, kn, ks, ko, workspace=torch.zeros(16, dtype=torch.uint8))
    with pytest.raises(abi.MixedGemmError):
        abi.fused_linear(x, idx, *good, kn, ks, ko, out=torch.zeros((m, n + 1), dtype=torch.bfloat16))


def test_matmul_refuses_short_scale_buffers_before_any_launch(no_launch):
    import torch
    abi = no_launch
    m, n, kn, ks, ko = 8, 64, 128, 64, 32
    u8 = dict(dtype=torch.uint8)
    b = _weights(abi, n, kn, ks, ko)
    a = [torch.zeros((m, kn // 2), **u8), torch.zeros((m, ks // 4 * 3), **u8), torch.zeros((m, ko), **u8),
         torch.zeros(abi.sf_bytes(m, kn, abi.MG_OPERAND_A), **u8), torch.zeros(abi.sf_bytes(m, ks, abi.MG_OPERAND_A), **u8),
         torch.zeros(abi.sf_bytes(m, ko, abi.MG_OPERAND_A), **u8)]

    def call(a, b):
        return abi.matmul(a[0], b[0], a[1], b[1], a[2], b[2], a[3], b[3], a[4], b[4], a[5], b[5])

    with pytest.raises(AssertionError, match="mg_mixed_gemm_ex reached"):
        call(a, b)
    for side, pos in (("a", 3), ("a", 4), ("a", 5), ("b", 3), ("b", 4), ("b", 5)):
        aa, bb = list(a), list(b)
        (aa if side == "a" else bb)[pos] = (aa if side == "a" else bb)[pos][:-1]
        with pytest.raises(abi.MixedGemmError, match="bytes, need"):
            call(aa, bb)


def test_the_binding_requires_gpu_tensors(abi):
    import torch
    m, n, kn, ks, ko = 8, 64, 128, 64, 32
    x = torch.zeros((m, kn + ks + ko), dtype=torch.bfloat16)
    idx = torch.arange(kn + ks + ko, dtype=torch.int16)
    with pytest.raises(abi.MixedGemmError, match="GPU tensor"):
        abi.fused_linear(x, idx, *_weights(abi, n, kn, ks, ko), kn, ks, ko)


def test_static_entry_point_refuses_what_does_not_fit(abi):
    lib = abi.lib()
    null = ctypes.c_void_p(0)
    # 8192 tokens at K = 4096 need 21 MB of quantized activations: more than the 20 MiB the library holds
    assert abi.fused_workspace_bytes(8192, 2560, 1408, 128) > abi.MG_STATIC_SCRATCH_BYTES
    assert lib.mg_fused_linear_static(*[null] * 8, 8192, 256, 2560, 1408, 128, 0, null, null) == 10005
    assert "static scratch" in abi.status_string(10005)
    # the benchmark configurations fit
    for m, kn, ks, ko in ((4096, 2560, 1408, 128), (2048, 8960, 4928, 448), (128, 2560, 1408, 128)):
        assert abi.fused_workspace_bytes(m, kn, ks, ko) <= abi.MG_STATIC_SCRATCH_BYTES
    # shape errors come first, empty problems succeed without touching the GPU
    assert lib.mg_fused_linear_static(*[null] * 8, 16, 256, 2560, 1400, 136, 0, null, null) == 10001
    assert lib.mg_fused_linear_static(*[null] * 8, 0, 256, 2560, 1408, 128, 0, null, null) == 0

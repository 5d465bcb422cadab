"""GPU parity for every shape bench.py times beyond the five benchmark configurations: the layer shapes
of the reference's K list (src/reorder.cu:508-576: 5120, 12288, 13824, 18944 next to 3584, 4096, 14336) at
the split `default_split` gives them -- segments that end 32, 64 or 96 channels past a whole 128-wide
stage at long K -- and the reference's own benchmark shape M=1024, N=4096, K=4096 (bench_gemm.cu:23-27,
bench_reorder_gemm.cu:143-169).  Quantize -> GEMM through the C-ABI against the oracle, row-major and
tile-major weights."""
import numpy as np
import pytest
import torch

from oracle import scalar as sc
from tests import helpers as H
from tests.test_gpu_parity import _check_gemm, _oracle_operands, _say

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def abi():
    from mixedgemm_amd import abi as a
    a.lib()
    return a


def _run_and_check(abi, m, n, kn, ks, ko, seed, what):
    k = kn + ks + ko
    x = H.make_activations(m, k, seed, n_out=max(1, k // 32))
    w = H.make_weights(n, k, seed + 1)
    idx = H.absmax_sort_index(x)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    aq = abi.reorder_quantize_x(xd, idd, kn, ks, ko)
    d_row = abi.matmul(aq[0], bq[0], aq[1], bq[1], aq[2], bq[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5])
    d_fused = abi.fused_linear(xd, idd, *bq, kn, ks, ko)
    torch.cuda.synchronize()
    H.assert_quant_equal(aq, sc.quantize_x(H.bf16_bits(x), idx.numpy(), kn, ks, ko), m, (kn, ks, ko), what=f"{what} x")
    H.assert_quant_equal(bq, sc.quantize_w(H.bf16_bits(w), idx.numpy(), kn, ks, ko), n, (kn, ks, ko), what=f"{what} w")
    qx, qw = _oracle_operands(x, w, idx, kn, ks, ko)
    _check_gemm(d_row, qx, qw, f"{what}, row-major weights")
    assert torch.equal(d_row, d_fused), f"{what}: fused call differs from quantize + GEMM"
    if abi.weights_tileable(n, kn, ks, ko):
        bt = abi.tile_weights(*bq[:3])
        d_tiled = abi.matmul(aq[0], bt[0], aq[1], bt[1], aq[2], bt[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5], w_tiled=True)
        d_tf = abi.fused_linear(xd, idd, bt[0], bt[1], bt[2], bq[3], bq[4], bq[5], kn, ks, ko, w_tiled=True)
        torch.cuda.synchronize()
        _check_gemm(d_tiled, qx, qw, f"{what}, tile-major weights")
        assert torch.equal(d_tiled, d_tf), f"{what}: fused call with tile-major weights differs"
        assert torch.equal(d_tiled, d_row), f"{what}: tile-major and row-major weights give different results"
    else:
        assert n % 256 != 0, f"{what}: a whole-tile shape that cannot be tiled"


@pytest.mark.parametrize("k", [5120, 12288, 13824, 18944, 3584, 14336])
@pytest.mark.parametrize("m,n", [(256, 256), (300, 512), (256, 512), (300, 256)])
def test_reference_k_list_at_the_default_split(abi, k, m, n):
    from mixedgemm_amd.linear import default_split
    kn, ks, ko = default_split(k)
    _say("bench shape", m, n, k, (kn, ks, ko))
    _run_and_check(abi, m, n, kn, ks, ko, 4000 + k + m + n, f"M={m} N={n} K={k} split {kn}/{ks}/{ko}")


def test_default_splits_are_the_ones_the_bench_times():
    from mixedgemm_amd.linear import default_split
    assert default_split(12288) == (7680, 4224, 384)
    assert default_split(13824) == (8576, 4800, 448)
    assert default_split(18944) == (11776, 6560, 608)
    assert default_split(5120) == (3200, 1760, 160)
    assert default_split(14336) == (8960, 4928, 448)


def test_reference_benchmark_shape(abi):
    """M=1024, N=4096, K=4096 (2560/1408/128): the problem bench_gemm.cu and bench_reorder_gemm.cu of the
    reference time.  64 tiles of 256 x 256."""
    m, n, kn, ks, ko = 1024, 4096, 2560, 1408, 128
    _say("reference bench shape", m, n, kn + ks + ko)
    _run_and_check(abi, m, n, kn, ks, ko, 8123, "reference bench shape")


@pytest.mark.parametrize("m,n,k,split", [
    (4096, 4096, 12288, None), (2048, 3584, 18944, None),
    # c3's M, N and K as pure E3M2 x E2M1 and E4M3 x E2M1 products (matmul_host6 / matmul_host8 of the reference on
    # their own: src/fp6.cu:35, src/fp8.cu:35) and without the E2M1 segment: the legs of bench.py's plans_without_a_segment
    (4096, 14336, 4096, (0, 4096, 0)), (4096, 14336, 4096, (0, 0, 4096)), (4096, 14336, 4096, (0, 3968, 128)),
])
def test_long_k_rows_of_the_shape_matrix_sampled(abi, m, n, k, split):
    """Rows of bench.py's shape matrix at (close to) full size: tile-major weights, sampled token rows
    against the oracle, every tile through the permutation property."""
    from mixedgemm_amd.linear import default_split
    from oracle import mx_oracle as mo
    kn, ks, ko = split or default_split(k)
    _say("shape matrix row", m, n, k, (kn, ks, ko))
    x = H.make_activations(m, k, 911 + k)
    w = H.make_weights(n, k, 913 + k)
    idx = H.absmax_sort_index(x)
    xd, wd, idd = x.to(DEV), w.to(DEV), idx.to(DEV)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    assert abi.weights_tileable(n, kn, ks, ko)
    bt = abi.tile_weights(*bq[:3]) + bq[3:]
    d = abi.fused_linear(xd, idd, *bt, kn, ks, ko, w_tiled=True)
    torch.cuda.synchronize()
    rng = np.random.default_rng(5)
    rows = np.sort(rng.choice(m, 24, replace=False))
    qx = mo.reorder_quantize_x(H.bf16_f32(x)[rows], idx.numpy(), kn, ks, ko)
    qw = mo.reorder_quantize_w(H.bf16_f32(w), idx.numpy(), kn, ks, ko)
    _check_gemm(d[torch.from_numpy(rows).to(DEV)], qx, qw, f"M={m} N={n} K={k} sampled rows")
    perm = torch.from_numpy(rng.permutation(m)).to(DEV)
    d_perm = abi.fused_linear(xd[perm].contiguous(), idd, *bt, kn, ks, ko, w_tiled=True)
    torch.cuda.synchronize()
    assert torch.equal(d_perm, d[perm])


# ------------------------------------------------------------------ reorder index range
def test_out_of_range_index_is_reported_and_clamped(abi):
    """mg_check_reorder_index names a bad index; the quantizer reads such an entry as channel K - 1 and
    stays inside the row."""
    rows, kn, ks, ko = 9, 128, 96, 32
    k = kn + ks + ko
    x = H.make_activations(rows, k, 77)
    idx = H.random_index(k, 78)
    abi.check_reorder_index(idx.to(DEV))
    bad = idx.clone()
    bad[5], bad[100], bad[200] = -3, k, 32767
    with pytest.raises(abi.MixedGemmError, match="out of range"):
        abi.check_reorder_index(bad.to(DEV))
    with pytest.raises(abi.MixedGemmError, match="out of range"):
        abi.check_reorder_index(bad)
    clamped = bad.clone()
    clamped[5], clamped[100], clamped[200] = k - 1, k - 1, k - 1
    got = abi.reorder_quantize_x(x.to(DEV), bad.to(DEV), kn, ks, ko)
    torch.cuda.synchronize()
    H.assert_quant_equal(got, sc.quantize_x(H.bf16_bits(x), clamped.numpy(), kn, ks, ko), rows, (kn, ks, ko), what="clamped index")

"""GPU tests of the caller layer: packed-weight file, registered torch operators on a side
stream, and the linear layer, against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as mo
from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def linear():
    from mixedgemm_amd import abi, linear as l
    abi.lib()
    return l


def _oracle_linear(x, w, idx, split):
    qx = mo.reorder_quantize_x(H.bf16_f32(x), idx.numpy(), *split)
    qw = mo.reorder_quantize_w(H.bf16_f32(w), idx.numpy(), *split)
    ref = mo.mixed_matmul(qx, qw)
    slack = (np.abs(mo.dequantize_x(qx)).astype(np.float64) @ np.abs(mo.dequantize_w(qw)).astype(np.float64).T) * 2.0 ** -20
    return ref, slack


def _close(d, ref, slack):
    err = np.abs(d.float().cpu().numpy() - mo.bf16_rne(ref))
    assert np.all(err <= H.bf16_ulp(ref) + slack), f"max err {err.max()}"


@pytest.mark.parametrize("m,n,k", [(24, 64, 4096), (3, 32, 3584), (256, 256, 5120)])
def test_linear_layer_matches_oracle(linear, m, n, k):
    print("linear layer", m, n, k, flush=True)
    split = linear.default_split(k)
    x = H.make_activations(m, k, 900 + m)
    w = H.make_weights(n, k, 901 + m)
    layer = linear.MixedLinear.from_float(w.to(DEV), calibration_x=x.to(DEV))
    idx = H.absmax_sort_index(x)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(layer.reorder_index.cpu().numpy(), idx.numpy())
    y = layer(x.to(DEV).reshape(1, m, k))
    torch.cuda.synchronize()
    assert y.shape == (1, m, n)
    ref, slack = _oracle_linear(x, w, idx, split)
    _close(y[0], ref, slack)


def test_pack_file_round_trip_through_the_gpu(linear, tmp_path):
    m, n, k = 16, 48, 4096
    split = linear.default_split(k)
    x = H.make_activations(m, k, 77)
    w = H.make_weights(n, k, 78)
    idx = H.absmax_sort_index(x)
    pw = linear.PackedWeights.from_float(w.to(DEV), idx.to(DEV), split)
    assert not pw.tiled          # 48 features: not a multiple of 256
    torch.cuda.synchronize()
    path = str(tmp_path / "layer.mgw")
    pw.save(path)
    back = linear.PackedWeights.load(path, device=DEV)
    assert not back.tiled
    for a, b in zip((*pw.tensors(), pw.reorder_index), (*back.tensors(), back.reorder_index)):
        assert torch.equal(a, b)
    y0 = linear.MixedLinear(pw)(x.to(DEV))
    y1 = linear.MixedLinear(back)(x.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(y0, y1)
    ref, slack = _oracle_linear(x, w, idx, split)
    _close(y1, ref, slack)


def test_operators_run_on_the_current_stream_without_synchronizing(linear):
    """The three reference calls as registered operators on a side stream: results are complete
    after waiting for that stream only, and equal those of the default stream."""
    m, n, k = 40, 64, 4096
    kn, ks, ko = linear.default_split(k)
    x = H.make_activations(m, k, 5).to(DEV)
    w = H.make_weights(n, k, 6).to(DEV)
    idx = torch.ops.mixedgemm_amd.calibrate_reorder_index(x)
    ops = torch.ops.mixedgemm_amd
    a = ops.reorder_quantize_x(x, idx, kn, ks, ko)
    b = ops.reorder_quantize_w(w, idx, kn, ks, ko)
    d0 = ops.matmul(a[0], b[0], a[1], b[1], a[2], b[2], a[3], b[3], a[4], b[4], a[5], b[5])
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        a1 = ops.reorder_quantize_x(x, idx, kn, ks, ko)
        d1 = ops.matmul(a1[0], b[0], a1[1], b[1], a1[2], b[2], a1[3], b[3], a1[4], b[4], a1[5], b[5])
        d2 = ops.fused_linear(x, idx, *b, kn, ks, ko)
    side.synchronize()
    assert torch.equal(d0, d1) and torch.equal(d0, d2)
    for t0, t1 in zip(a[:3], a1[:3]):
        assert torch.equal(t0, t1)


@pytest.mark.parametrize("m", [8, 300])
def test_tiled_pack_round_trip_and_layer(linear, tmp_path, m):
    """Default packing of a tileable layer is tile-major; the file keeps the layout and the layer gives
    the row-major result bit for bit."""
    n, k = 512, 4096
    split = linear.default_split(k)
    x = H.make_activations(m, k, 81)
    w = H.make_weights(n, k, 82)
    idx = H.absmax_sort_index(x)
    tiled = linear.PackedWeights.from_float(w.to(DEV), idx.to(DEV), split)
    plain = linear.PackedWeights.from_float(w.to(DEV), idx.to(DEV), split, tile=False)
    assert tiled.tiled and not plain.tiled and not torch.equal(tiled.wn, plain.wn)
    path = str(tmp_path / "tiled.mgw")
    tiled.save(path)
    assert linear.read_header(path)[0]["code_layout"] == "tile-major-256x128"
    back = linear.PackedWeights.load(path, device=DEV)
    assert back.tiled and torch.equal(back.wn, tiled.wn) and torch.equal(back.ws, tiled.ws)
    y0 = linear.MixedLinear(plain)(x.to(DEV))
    y1 = linear.MixedLinear(back)(x.to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(y0, y1)
    ref, slack = _oracle_linear(x, w, idx, split)
    _close(y1, ref, slack)


def test_layer_with_fused_rmsnorm(linear):
    m, n, k, eps = 70, 256, 4096, 1e-5
    split = linear.default_split(k)
    x = H.make_activations(m, k, 91)
    w = H.make_weights(n, k, 92)
    g = torch.Generator().manual_seed(93)
    gamma = (torch.randn(k, generator=g) * 0.3 + 1.0).to(torch.bfloat16)
    y = torch.from_numpy(mo.rmsnorm_bf16(H.bf16_bits(x), H.bf16_bits(gamma), eps).view(np.int16)).view(torch.bfloat16)
    idx = H.absmax_sort_index(y)
    pw = linear.PackedWeights.from_float(w.to(DEV), idx.to(DEV), split)
    layer = linear.MixedLinear(pw, norm_weight=gamma.to(DEV), eps=eps)
    out = layer(x.to(DEV))
    torch.cuda.synchronize()
    ref, slack = _oracle_linear(y, w, idx, split)
    _close(out, ref, slack)


def test_layer_replayed_as_a_hip_graph(linear):
    """The whole layer (RMSNorm + reorder-quantize + GEMM: three of our launches, nothing else) captured once
    and replayed with new inputs in the same buffers; every replay must equal the eager result."""
    m, n, k = 300, 512, 4096
    split = linear.default_split(k)
    g = torch.Generator().manual_seed(7)
    gamma = (torch.randn(k, generator=g) * 0.3 + 1.0).to(torch.bfloat16).to(DEV)
    xs = [H.make_activations(m, k, 200 + i).to(DEV) for i in range(3)]
    w = H.make_weights(n, k, 210).to(DEV)
    from mixedgemm_amd import abi
    idx = abi.calibrate_reorder_index(xs[0])
    pw = linear.PackedWeights.from_float(w, idx, split)
    x_buf = xs[0].clone()
    ws = torch.empty(abi.fused_workspace_bytes(m, *split), dtype=torch.uint8, device=DEV)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)

    def run():
        abi.fused_linear(x_buf, idx, *pw.tensors(), *split, workspace=ws, out=out, w_tiled=pw.tiled,
                         norm_weight=gamma, eps=1e-5)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        run()                                # warm-up outside the capture (first-call setup)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            run()
    torch.cuda.synchronize()
    for i in (1, 2, 0, 1):
        x_buf.copy_(xs[i])
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = abi.fused_linear(xs[i], idx, *pw.tensors(), *split, w_tiled=pw.tiled, norm_weight=gamma, eps=1e-5)
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay with input {i} differs from the eager result"


@pytest.mark.parametrize("m,n", [(300, 1000), (8, 300)])
def test_layer_pads_odd_feature_counts_to_whole_tiles(linear, tmp_path, m, n):
    """N that is not a multiple of 256: the packer appends zero rows so that the whole-tile kernel and
    tile-major weights apply; the layer returns the real N columns, and the file keeps both counts."""
    k = 4096
    split = linear.default_split(k)
    x = H.make_activations(m, k, 95)
    w = H.make_weights(n, k, 96)
    idx = H.absmax_sort_index(x)
    pw = linear.PackedWeights.from_float(w.to(DEV), idx.to(DEV), split)
    assert pw.out_features == n and pw.rows % 256 == 0 and pw.rows >= n and pw.tiled
    path = str(tmp_path / "odd.mgw")
    pw.save(path)
    back = linear.PackedWeights.load(path, device=DEV)
    assert back.out_features == n and back.rows == pw.rows and back.tiled
    y = linear.MixedLinear(back)(x.to(DEV))
    torch.cuda.synchronize()
    assert y.shape == (m, n)
    ref, slack = _oracle_linear(x, w, idx, split)
    _close(y, ref, slack)


@pytest.mark.parametrize("split", [(512, 0, 0), (384, 0, 128), (384, 128, 0)])
def test_layer_with_a_plan_that_has_no_e3m2_or_e4m3_segment(linear, tmp_path, split):
    """All-MXFP4 activations, MXFP4 + MXFP8 outliers, MXFP4 + MXFP6: packed tile-major, saved, loaded, run."""
    m, n, k = 300, 512, sum(split)
    x = H.make_activations(m, k, 97, n_out=8)
    w = H.make_weights(n, k, 98)
    idx = H.absmax_sort_index(x)
    pw = linear.PackedWeights.from_float(w.to(DEV), idx.to(DEV), split)
    assert pw.tiled
    path = str(tmp_path / "partial.mgw")
    pw.save(path)
    back = linear.PackedWeights.load(path, device=DEV)
    assert back.split == tuple(split) and back.tiled
    y = linear.MixedLinear(back)(x.to(DEV))
    torch.cuda.synchronize()
    ref, slack = _oracle_linear(x, w, idx, split)
    _close(y, ref, slack)

"""mg_fused_linear_static -- the fused entry point that allocates nothing and keeps the quantized
activations in the library's own static device array -- against mg_fused_linear_ex with a caller
workspace: bit-identical outputs, on calls in a row that share the array (the later ones smaller, so
that what an earlier call left behind lies next to what they use)."""
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def abi():
    from mixedgemm_amd import abi as a
    a.lib()
    return a


def _problem(abi, m, n, kn, ks, ko, seed, tile):
    k = kn + ks + ko
    x = H.make_activations(m, k, seed).to(DEV)
    w = H.make_weights(n, k, seed + 1).to(DEV)
    idx = H.absmax_sort_index(x.cpu()).to(DEV)
    bq = abi.reorder_quantize_w(w, idx, kn, ks, ko)
    if tile:
        assert abi.weights_tileable(n, kn, ks, ko)
        bq = abi.tile_weights(*bq[:3]) + bq[3:]
    return x, idx, bq


def _both(abi, x, idx, bq, split, tile):
    m, n = x.shape[0], bq[0].shape[0]
    want = abi.fused_linear(x, idx, *bq, *split, w_tiled=tile)
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    # an untimed first call: the library looks up its scratch array's address once per device
    abi.fused_linear_static(x, idx, *bq, *split, out=got, w_tiled=tile)
    torch.cuda.synchronize()
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    # neither torch's allocator nor the driver hands out or takes back device memory during the call
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    abi.fused_linear_static(x, idx, *bq, *split, out=got, w_tiled=tile)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    return got, want


@pytest.mark.parametrize("first,second,split,tile", [
    ((512, 512), (300, 512), (2560, 1408, 128), True),      # whole-tile kernel, then a ragged last tile
    ((300, 256), (40, 256), (448, 416, 224), False),        # whole-tile kernel, then the skinny one
    ((64, 1000), (8, 1000), (2560, 1408, 128), False),      # decode sizes
])
def test_static_scratch_entry_point_matches_the_workspace_one(abi, first, second, split, tile):
    print("no-alloc", first, second, split, tile, flush=True)
    outs = []
    for i, (m, n) in enumerate((first, second, first)):
        x, idx, bq = _problem(abi, m, n, *split, 600 + 10 * i + m, tile)
        got, want = _both(abi, x, idx, bq, split, tile)
        assert torch.equal(got, want), f"call {i} ({m} x {n}): static-scratch result differs from the workspace one"
        outs.append(got)
    assert not torch.isnan(outs[1].float()).any()


def test_static_scratch_at_the_largest_benchmark_configuration(abi):
    """c3's activations (4096 x 4096) fill 10.6 MB of the 20 MiB array; a narrow weight matrix keeps the test short."""
    split = (2560, 1408, 128)
    x, idx, bq = _problem(abi, 4096, 512, *split, 700, True)
    got, want = _both(abi, x, idx, bq, split, True)
    assert torch.equal(got, want)
    x2, idx2, bq2 = _problem(abi, 1000, 512, *split, 701, True)
    got2, want2 = _both(abi, x2, idx2, bq2, split, True)
    assert torch.equal(got2, want2)


def test_static_scratch_refuses_what_does_not_fit(abi):
    split = (2560, 1408, 128)
    x, idx, bq = _problem(abi, 8, 256, *split, 702, False)
    big = torch.zeros((8192, sum(split)), dtype=torch.bfloat16, device=DEV)
    out = torch.empty((8192, 256), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(abi.MixedGemmError, match="static scratch"):
        abi.fused_linear_static(big, idx, *bq, *split, out=out)

"""Host-side pieces of the caller layer that need no GPU: the K split, the packed-weight file,
and the shape functions of the registered torch operators."""
import numpy as np
import pytest
import torch

from mixedgemm_amd import abi, linear


def test_default_split_reproduces_the_reference_splits():
    assert linear.default_split(4096) == (2560, 1408, 128)      # bench_reorder.cu:26-28
    assert linear.default_split(3584) == (2560, 896, 128)       # main.py:9
    assert linear.default_split(14336) == (8960, 4928, 448)     # the down-projection configuration


@pytest.mark.parametrize("k", linear.REFERENCE_K)
def test_default_split_is_usable_for_every_reference_k(k):
    kn, ks, ko = linear.default_split(k)
    assert kn + ks + ko == k and min(kn, ks, ko) >= 128
    assert kn % 128 == 0 and ks % 32 == 0 and ko % 32 == 0
    if k != 3584:   # main.py:9 keeps the K=4096 MXFP4 share for its 3584-channel example
        assert abs(ko / k - 1 / 32) < 0.003 and abs(kn / k - 5 / 8) < 0.01


def test_default_split_rejects_odd_k():
    with pytest.raises(ValueError):
        linear.default_split(4100)


def _random_pack(n, split, seed=0):
    g = torch.Generator().manual_seed(seed)
    kn, ks, ko = split
    u8 = lambda *shape: torch.randint(0, 256, shape, dtype=torch.uint8, generator=g)
    return linear.PackedWeights(
        u8(n, kn // 2), u8(n, ks // 2), u8(n, ko // 2),
        u8(abi.sf_bytes(n, kn, abi.MG_OPERAND_B)), u8(abi.sf_bytes(n, ks, abi.MG_OPERAND_B)),
        u8(abi.sf_bytes(n, ko, abi.MG_OPERAND_B)),
        torch.randperm(sum(split), generator=g).to(torch.int16), split)


@pytest.mark.parametrize("n,split", [(5, (256, 128, 128)), (130, (2560, 896, 128)), (3, (128, 0, 0))])
def test_pack_file_round_trip(tmp_path, n, split):
    pw = _random_pack(n, split)
    path = str(tmp_path / "layer.mgw")
    pw.save(path)
    header, data_offset = linear.read_header(path)
    assert header["split"] == list(split) and header["out_features"] == n and data_offset % 256 == 0
    assert all(s["offset"] % 256 == 0 for s in header["sections"].values())
    back = linear.PackedWeights.load(path)
    assert back.split == split
    for a, b in zip((*pw.tensors(), pw.reorder_index), (*back.tensors(), back.reorder_index)):
        assert a.dtype == b.dtype and torch.equal(a, b)


def test_pack_file_rejects_foreign_and_truncated_files(tmp_path):
    bad = tmp_path / "x.bin"
    bad.write_bytes(b"not a pack file at all")
    with pytest.raises(ValueError):
        linear.PackedWeights.load(str(bad))
    pw = _random_pack(4, (256, 128, 128))
    path = tmp_path / "layer.mgw"
    pw.save(str(path))
    data = path.read_bytes()
    (tmp_path / "short.mgw").write_bytes(data[:len(data) - 300])
    with pytest.raises(ValueError):
        linear.PackedWeights.load(str(tmp_path / "short.mgw"))


def test_validate_catches_wrong_shapes():
    pw = _random_pack(4, (256, 128, 128))
    pw.ws = pw.ws[:, :-1]
    with pytest.raises(ValueError):
        pw.validate()


def test_operator_shape_functions():
    """The registered fake kernels give the reference's output shapes (bindings.cpp:30-36,85-93,204-212)."""
    m, n, (kn, ks, ko) = 130, 24, (256, 128, 128)
    k = kn + ks + ko
    X = torch.empty((m, k), dtype=torch.bfloat16, device="meta")
    W = torch.empty((n, k), dtype=torch.bfloat16, device="meta")
    idx = torch.empty((k,), dtype=torch.int16, device="meta")
    a = torch.ops.mixedgemm_amd.reorder_quantize_x(X, idx, kn, ks, ko)
    b = torch.ops.mixedgemm_amd.reorder_quantize_w(W, idx, kn, ks, ko)
    assert [tuple(t.shape) for t in a[:3]] == [(m, kn // 2), (m, ks // 4 * 3), (m, ko)]
    assert [tuple(t.shape) for t in b[:3]] == [(n, kn // 2), (n, ks // 2), (n, ko // 2)]
    assert [t.numel() for t in a[3:]] == [(m // 128 + 1) * 128 * s // 32 for s in (kn, ks, ko)]
    assert [t.numel() for t in b[3:]] == [abi.sf_bytes(n, s, abi.MG_OPERAND_B) for s in (kn, ks, ko)]
    d = torch.ops.mixedgemm_amd.matmul(a[0], b[0], a[1], b[1], a[2], b[2], a[3], b[3], a[4], b[4], a[5], b[5])
    assert d.shape == (m, n) and d.dtype == torch.bfloat16
    d = torch.ops.mixedgemm_amd.fused_linear(X, idx, *b, kn, ks, ko)
    assert d.shape == (m, n) and d.dtype == torch.bfloat16
    assert torch.ops.mixedgemm_amd.calibrate_reorder_index(X).shape == (k,)


def test_operators_refuse_cpu_tensors():
    """No CPU fallback: a host tensor is an error, not a slow path."""
    x = torch.zeros((4, 128), dtype=torch.bfloat16)
    idx = torch.arange(128, dtype=torch.int16)
    with pytest.raises(abi.MixedGemmError):
        torch.ops.mixedgemm_amd.reorder_quantize_x(x, idx, 128, 0, 0)


def test_validate_rejects_an_index_outside_the_channels_and_mixed_devices():
    import pytest
    import torch
    from mixedgemm_amd import abi
    from mixedgemm_amd.linear import PackedWeights
    n, split = 16, (64, 32, 32)
    k = sum(split)
    u8 = dict(dtype=torch.uint8)
    def make(idx):
        return PackedWeights(torch.zeros((n, 32), **u8), torch.zeros((n, 16), **u8), torch.zeros((n, 16), **u8),
                             torch.zeros(abi.sf_bytes(n, 64, abi.MG_OPERAND_B), **u8),
                             torch.zeros(abi.sf_bytes(n, 32, abi.MG_OPERAND_B), **u8),
                             torch.zeros(abi.sf_bytes(n, 32, abi.MG_OPERAND_B), **u8), idx, split)
    make(torch.arange(k, dtype=torch.int16)).validate()
    for pos, val in ((0, -1), (5, k), (k - 1, 4000)):
        idx = torch.arange(k, dtype=torch.int16)
        idx[pos] = val
        with pytest.raises(ValueError, match="out of range"):
            make(idx).validate()
    pw = make(torch.arange(k, dtype=torch.int16))
    pw.sfwo = pw.sfwo.to("meta")
    with pytest.raises(ValueError, match="different devices"):
        pw.validate()

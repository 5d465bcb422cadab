"""The C-ABI without torch: build/abi_driver (tests/c_host/abi_driver.cpp: HIP runtime + the library's
extern "C" entry points) runs the whole path on a problem file; its outputs are compared with the golden
vectors and with the oracle."""
import glob
import os
import subprocess

import numpy as np
import pytest

from oracle import mx_oracle as mo
from oracle import scalar as sc
from tests import helpers as H

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "build", "abi_driver")
GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "path_*.npz")))


def _sf_bytes(rows, kseg, operand):
    return mo.sf_bytes(rows, kseg, operand)


def _run(tmp_path, x_bits, w_bits, split):
    assert os.path.exists(DRIVER), "build/abi_driver is missing: python -m mixedgemm_amd.build"
    m, k = x_bits.shape
    n = w_bits.shape[0]
    kn, ks, ko = split
    src, dst = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(src, "wb") as f:
        f.write(np.array([m, n, kn, ks, ko], np.int32).tobytes())
        f.write(np.ascontiguousarray(x_bits).tobytes())
        f.write(np.ascontiguousarray(w_bits).tobytes())
    r = subprocess.run([DRIVER, src, dst], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stderr
    raw = np.fromfile(dst, dtype=np.uint8)
    pos = 0

    def take(nbytes):
        nonlocal pos
        out = raw[pos:pos + nbytes]
        pos += nbytes
        return out

    idx = take(2 * k).view(np.int16)
    a_sizes = [m * kn // 2, m * ks // 4 * 3, m * ko] + [_sf_bytes(m, s, "a") for s in split]
    b_sizes = [n * kn // 2, n * ks // 2, n * ko // 2] + [_sf_bytes(n, s, "b") for s in split]
    a = [take(s) for s in a_sizes]
    b = [take(s) for s in b_sizes]
    d1 = take(2 * m * n).view(np.uint16).reshape(m, n)
    d2 = take(2 * m * n).view(np.uint16).reshape(m, n)
    assert pos == raw.size
    return idx, a, b, d1, d2


def _bf16_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def _check_d(bits, ref, slack, what):
    err = np.abs(_bf16_to_f32(bits) - mo.bf16_rne(ref))
    assert np.all(err <= H.bf16_ulp(ref) + slack), f"{what}: max err {err.max()}"


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_c_host_program_reproduces_golden_vectors(tmp_path, path):
    g = np.load(path)
    split = tuple(int(v) for v in g["split"])
    idx, a, b, d1, d2 = _run(tmp_path, g["x_bits"], g["w_bits"], split)
    m, n = g["x_bits"].shape[0], g["w_bits"].shape[0]
    np.testing.assert_array_equal(idx, g["idx"])
    for tag, bufs, rows in (("x", a, m), ("w", b, n)):
        for buf, c in zip(bufs[:3], ("qn", "qs", "qo")):
            np.testing.assert_array_equal(buf, g[f"{tag}_{c}"].reshape(-1), err_msg=f"{tag} {c}")
        for buf, s, kseg in zip(bufs[3:], ("sfn", "sfs", "sfo"), split):
            np.testing.assert_array_equal(mo.sf_gather(buf, rows, kseg), g[f"{tag}_{s}"], err_msg=f"{tag} {s}")
    slack = g["d_abs_f32"] * 2.0 ** -20
    _check_d(d1, g["d_f32"], slack, "mg_mixed_gemm")
    _check_d(d2, g["d_f32"], slack, "mg_fused_linear_ex")


def test_c_host_program_on_a_ragged_prefill_shape_with_tiled_weights(tmp_path):
    """300 tokens x 512 features from hipMalloc'ed exact-size buffers: the last token tile of the plain GEMM reads
    no row past the 300th; the fused call runs the same tiles on its padded workspace, with tile-major weights."""
    m, n, split = 300, 512, (2560, 1408, 128)
    k = sum(split)
    x = H.make_activations(m, k, 501)
    w = H.make_weights(n, k, 502)
    idx, a, b, d1, d2 = _run(tmp_path, H.bf16_bits(x), H.bf16_bits(w), split)
    ref_idx = H.absmax_sort_index(x).numpy()
    np.testing.assert_array_equal(idx, ref_idx)
    qx = sc.quantize_x(H.bf16_bits(x), ref_idx, *split)
    qw = sc.quantize_w(H.bf16_bits(w), ref_idx, *split)
    for buf, c in zip(a[:3], ("qn", "qs", "qo")):
        np.testing.assert_array_equal(buf, qx[c].reshape(-1))
    for buf, c in zip(b[:3], ("qn", "qs", "qo")):
        np.testing.assert_array_equal(buf, qw[c].reshape(-1))
    fx = mo.reorder_quantize_x(H.bf16_f32(x), ref_idx, *split)
    fw = mo.reorder_quantize_w(H.bf16_f32(w), ref_idx, *split)
    ref = mo.mixed_matmul(fx, fw)
    slack = (np.abs(mo.dequantize_x(fx)).astype(np.float64) @ np.abs(mo.dequantize_w(fw)).astype(np.float64).T) * 2.0 ** -20
    _check_d(d1, ref, slack, "mg_mixed_gemm")
    _check_d(d2, ref, slack, "mg_fused_linear_ex, tile-major weights")

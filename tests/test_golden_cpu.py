"""Both CPU restatements against the committed golden vectors of the whole path
(tests/golden/path_*.npz, written by tests/golden/make_fixtures.py)."""
import glob
import os

import numpy as np
import pytest

from oracle import mx_oracle as mo
from oracle import scalar as sc

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "path_*.npz")))


def bits_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def test_fixtures_present():
    assert len(GOLDEN) == 3


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_oracles_reproduce_golden_vectors(path):
    g = np.load(path)
    kn, ks, ko = (int(v) for v in g["split"])
    idx = g["idx"]
    for tag, bits, scalar_fn, numpy_fn in (("x", g["x_bits"], sc.quantize_x, mo.reorder_quantize_x),
                                           ("w", g["w_bits"], sc.quantize_w, mo.reorder_quantize_w)):
        rows = bits.shape[0]
        for q in (scalar_fn(bits, idx, kn, ks, ko), numpy_fn(bits_to_f32(bits), idx, kn, ks, ko)):
            for c in ("qn", "qs", "qo"):
                np.testing.assert_array_equal(q[c], g[f"{tag}_{c}"], err_msg=f"{tag} {c}")
            for s, kseg in zip(("sfn", "sfs", "sfo"), (kn, ks, ko)):
                np.testing.assert_array_equal(mo.sf_gather(q[s], rows, kseg), g[f"{tag}_{s}"], err_msg=f"{tag} {s}")
    qx = mo.reorder_quantize_x(bits_to_f32(g["x_bits"]), idx, kn, ks, ko)
    qw = mo.reorder_quantize_w(bits_to_f32(g["w_bits"]), idx, kn, ks, ko)
    np.testing.assert_array_equal(mo.mixed_matmul(qx, qw).astype(np.float32), g["d_f32"])


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_golden_index_is_the_calibrated_one(path):
    g = np.load(path)
    np.testing.assert_array_equal(mo.calibrate_reorder_index(g["x_bits"]), g["idx"])

"""Caller side of the path: the K split, the packed-weight file, stream-ordered torch operators
and a linear layer on top of them.

The reference leaves all of this to the script that drives it (main.py:8-9 picks the split,
main.py:31-33 sketches the calibration, main.py:36 re-quantizes the weights on every run and
every operator ends in a device-wide synchronize, bindings.cpp:59,178,297).  Here the weights
are quantized once and kept (in memory or in a file), and every operator only enqueues work on
torch's current stream.
"""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass

import numpy as np
import torch

from . import abi

# Channels per K as the reference instantiates its quantizers (reorder.cu:508-576); the split of
# 3584 is the one main.py:9 uses, 4096 the one of bench_reorder.cu:26-28.  Every other K takes the
# same proportions as 4096 (5/8 MXFP4 rounded down to whole 128-channel MFMA steps, 1/32 MXFP8
# rounded up to whole 32-channel scale blocks, the rest MXFP6); 14336 gives 8960/4928/448.
REFERENCE_K = (4096, 5120, 3584, 14336, 18944, 12288, 13824)
_SPLITS = {3584: (2560, 896, 128), 4096: (2560, 1408, 128)}


def default_split(k: int) -> tuple[int, int, int]:
    """(KN, KS, KO) for a layer with k input channels."""
    if k in _SPLITS:
        return _SPLITS[k]
    if k % 32 or k < 1024:
        raise ValueError(f"K={k}: the default split needs a multiple of 32, at least 1024")
    ko = max(128, (k // 32 + 31) // 32 * 32)
    kn = k * 5 // 8 // 128 * 128
    return kn, k - kn - ko, ko


# ------------------------------------------------------------------ packed weights
MAGIC = b"MGWPACK1"
_ALIGN = 256
_SECTIONS = ("wn", "ws", "wo", "sfwn", "sfws", "sfwo", "reorder_index")


@dataclass
class PackedWeights:
    """One layer's weights after reorder-quantize: three code tensors (all E2M1, two per byte),
    three E8M0 scale buffers in the GEMM's interleaved layout, the reorder index the activations
    must be gathered with, and the split."""
    wn: torch.Tensor
    ws: torch.Tensor
    wo: torch.Tensor
    sfwn: torch.Tensor
    sfws: torch.Tensor
    sfwo: torch.Tensor
    reorder_index: torch.Tensor
    split: tuple[int, int, int]
    tiled: bool = False   # wn, ws, wo in the tile-major order of mg_tile_weights (same shapes)
    features: int = 0     # output features that are real; 0 = every stored row (rows past it are zero padding)

    @property
    def rows(self) -> int:
        """Stored weight rows (a multiple of 256 when the layer was padded for the whole-tile kernel)."""
        return self.wn.shape[0] if self.split[0] else (self.ws.shape[0] if self.split[1] else self.wo.shape[0])

    @property
    def out_features(self) -> int:
        return self.features or self.rows

    @property
    def in_features(self) -> int:
        return sum(self.split)

    def tensors(self):
        return self.wn, self.ws, self.wo, self.sfwn, self.sfws, self.sfwo

    @classmethod
    def from_float(cls, weight: torch.Tensor, reorder_index: torch.Tensor, split=None, tile=True) -> "PackedWeights":
        """Quantizes bf16 weight[N, K] on its GPU (reorder_quantize_w of the reference,
        bindings.cpp:188-305); with `tile`, shapes that allow it are then put in tile-major order."""
        split = tuple(split) if split is not None else default_split(weight.shape[1])
        n = weight.shape[0]
        abi.check_reorder_index(reorder_index, weight.shape[1])
        # the whole-tile kernel wants a multiple of 256 features: zero rows are cheap, the layer drops their outputs
        if tile and n > 256 and n % 256 and abi.weights_tileable((n + 255) // 256 * 256, *split):
            pad = torch.zeros(((n + 255) // 256 * 256 - n, weight.shape[1]), dtype=weight.dtype, device=weight.device)
            weight = torch.cat([weight, pad])
        q = abi.reorder_quantize_w(weight, reorder_index, *split)
        pw = cls(*q, reorder_index, split, False, n if weight.shape[0] != n else 0)
        return pw.tile() if tile and pw.tileable() else pw

    def tileable(self) -> bool:
        return abi.weights_tileable(self.rows, *self.split)

    def tile(self) -> "PackedWeights":
        """The same weights with the codes in tile-major order (GPU tensors).  The prefill kernel
        copies them 10-15 % faster; the decode kernel a few percent slower."""
        if self.tiled:
            return self
        if not self.tileable():
            raise ValueError("tile-major order needs N % 256 == 0 and a split the whole-tile kernel takes (abi.weights_tileable)")
        wn, ws, wo = abi.tile_weights(self.wn, self.ws, self.wo)
        return PackedWeights(wn, ws, wo, self.sfwn, self.sfws, self.sfwo, self.reorder_index, self.split, True, self.features)

    def to(self, device) -> "PackedWeights":
        return PackedWeights(*(t.to(device) for t in self.tensors()), self.reorder_index.to(device), self.split, self.tiled,
                             self.features)

    # The file: MAGIC, u32 header length, u32 data offset, JSON header, then at the data offset
    # (a multiple of 256) the sections, each at a 256-byte aligned offset counted from there.
    # Scale buffers are stored as the GEMM reads them, so loading is a plain copy to the device.
    def save(self, path: str) -> None:
        arrays = {name: t.detach().cpu().contiguous().numpy()
                  for name, t in zip(_SECTIONS, (*self.tensors(), self.reorder_index))}
        header = {"format": "mixedgemm-packed-weights", "version": 1, "out_features": self.out_features,
                  "stored_rows": self.rows,
                  "in_features": self.in_features, "split": list(self.split),
                  "scale_layout": "128x4-interleaved-e8m0",
                  "code_layout": "tile-major-256x128" if self.tiled else "row-major", "sections": {}}
        pos = 0
        for name in _SECTIONS:
            a = arrays[name]
            header["sections"][name] = {"offset": pos, "nbytes": int(a.nbytes), "shape": list(a.shape), "dtype": str(a.dtype)}
            pos = _round_up(pos + a.nbytes, _ALIGN)
        blob = json.dumps(header, sort_keys=True).encode()
        data_offset = _round_up(len(MAGIC) + 8 + len(blob), _ALIGN)
        tmp = path + ".tmp"
        with open(tmp, "wb") as f:
            f.write(MAGIC + struct.pack("<II", len(blob), data_offset) + blob)
            for name in _SECTIONS:
                f.seek(data_offset + header["sections"][name]["offset"])
                f.write(arrays[name].tobytes())
            f.truncate(data_offset + pos)
        os.replace(tmp, path)

    @classmethod
    def load(cls, path: str, device="cpu") -> "PackedWeights":
        header, data_offset = read_header(path)
        m = np.memmap(path, dtype=np.uint8, mode="r")
        out = []
        for name in _SECTIONS:
            s = header["sections"][name]
            dt = np.dtype(s["dtype"])
            if dt != (np.int16 if name == "reorder_index" else np.uint8):
                raise ValueError(f"{path}: section {name} has dtype {dt}")
            if data_offset + s["offset"] + s["nbytes"] > m.size or s["nbytes"] != int(np.prod(s["shape"])) * dt.itemsize:
                raise ValueError(f"{path}: section {name} does not fit the file")
            a = np.frombuffer(m, dtype=dt, count=s["nbytes"] // dt.itemsize, offset=data_offset + s["offset"])
            out.append(torch.from_numpy(np.array(a).reshape(s["shape"])).to(device))
        split = tuple(int(v) for v in header["split"])
        layout = header.get("code_layout", "row-major")
        if layout not in ("row-major", "tile-major-256x128"):
            raise ValueError(f"{path}: unknown code layout {layout}")
        n_real = int(header.get("out_features", 0))
        pw = cls(*out, split, layout != "row-major")
        pw.features = n_real if n_real != pw.rows else 0
        pw.validate()
        return pw

    def validate(self) -> None:
        kn, ks, ko = self.split
        n = self.rows
        if not 0 <= self.features <= n:
            raise ValueError(f"{self.features} real features in {n} stored rows")
        want = {"wn": (n, kn // 2), "ws": (n, ks // 2), "wo": (n, ko // 2)}
        for name, shape in want.items():
            t = getattr(self, name)
            if tuple(t.shape) != shape or t.dtype != torch.uint8:
                raise ValueError(f"{name}: expected uint8 {shape}, got {t.dtype} {tuple(t.shape)}")
        for name, kseg in (("sfwn", kn), ("sfws", ks), ("sfwo", ko)):
            t = getattr(self, name)
            need = abi.sf_bytes(n, kseg, abi.MG_OPERAND_B)
            if t.dtype != torch.uint8 or t.numel() < need:
                raise ValueError(f"{name}: expected at least {need} uint8, got {t.numel()} {t.dtype}")
        if self.reorder_index.dtype != torch.int16 or self.reorder_index.numel() != kn + ks + ko:
            raise ValueError("reorder_index: expected int16 [K]")
        devices = {t.device for t in (*self.tensors(), self.reorder_index)}
        if len(devices) != 1:
            raise ValueError(f"tensors on different devices: {sorted(str(d) for d in devices)}")
        try:
            abi.check_reorder_index(self.reorder_index.contiguous(), kn + ks + ko)   # blocks for GPU tensors: a pack-time check
        except abi.MixedGemmError as e:
            raise ValueError(str(e)) from e
        if self.tiled and not self.tileable():
            raise ValueError("tile-major codes for a shape that cannot be tiled")


def _round_up(v: int, a: int) -> int:
    return (v + a - 1) // a * a


def read_header(path: str):
    """(header dict, offset of the data area)."""
    with open(path, "rb") as f:
        if f.read(len(MAGIC)) != MAGIC:
            raise ValueError(f"{path}: not a packed-weight file")
        n, data_offset = struct.unpack("<II", f.read(8))
        header = json.loads(f.read(n).decode())
    if header.get("version") != 1:
        raise ValueError(f"{path}: unsupported version {header.get('version')}")
    return header, data_offset


# ------------------------------------------------------------------ torch operators
# Same names and argument order as the reference's module (bindings.cpp:315-341), in the
# namespace mixedgemm_amd; they enqueue on the current stream and return without synchronizing.
def _sf_len(rows: int, kseg: int, operand: int) -> int:
    return abi.sf_bytes(rows, kseg, operand)


@torch.library.custom_op("mixedgemm_amd::reorder_quantize_x", mutates_args=())
def reorder_quantize_x_op(X: torch.Tensor, reorder_index: torch.Tensor, KN: int, KS: int, KO: int
                          ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    return abi.reorder_quantize_x(X, reorder_index, KN, KS, KO)


@torch.library.custom_op("mixedgemm_amd::reorder_quantize_w", mutates_args=())
def reorder_quantize_w_op(W: torch.Tensor, reorder_index: torch.Tensor, KN: int, KS: int, KO: int
                          ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    return abi.reorder_quantize_w(W, reorder_index, KN, KS, KO)


def _fake_quant(operand):
    def fake(T, reorder_index, KN, KS, KO):
        rows = T.shape[0]
        w = operand == abi.MG_OPERAND_B
        u8 = dict(dtype=torch.uint8, device=T.device)
        return (torch.empty((rows, KN // 2), **u8),
                torch.empty((rows, KS // 2 if w else KS // 4 * 3), **u8),
                torch.empty((rows, KO // 2 if w else KO), **u8),
                torch.empty(_sf_len(rows, KN, operand), **u8),
                torch.empty(_sf_len(rows, KS, operand), **u8),
                torch.empty(_sf_len(rows, KO, operand), **u8))
    return fake


reorder_quantize_x_op.register_fake(_fake_quant(abi.MG_OPERAND_A))
reorder_quantize_w_op.register_fake(_fake_quant(abi.MG_OPERAND_B))


@torch.library.custom_op("mixedgemm_amd::matmul", mutates_args=())
def matmul_op(AN: torch.Tensor, BN: torch.Tensor, AS: torch.Tensor, BS: torch.Tensor, AO: torch.Tensor, BO: torch.Tensor,
              SFAN: torch.Tensor, SFBN: torch.Tensor, SFAS: torch.Tensor, SFBS: torch.Tensor, SFAO: torch.Tensor,
              SFBO: torch.Tensor, w_tiled: bool = False) -> torch.Tensor:
    return abi.matmul(AN, BN, AS, BS, AO, BO, SFAN, SFBN, SFAS, SFBS, SFAO, SFBO, w_tiled=w_tiled)


@matmul_op.register_fake
def _(AN, BN, AS, BS, AO, BO, SFAN, SFBN, SFAS, SFBS, SFAO, SFBO, w_tiled=False):
    return torch.empty((AN.shape[0], BN.shape[0]), dtype=torch.bfloat16, device=AN.device)


@torch.library.custom_op("mixedgemm_amd::fused_linear", mutates_args=())
def fused_linear_op(X: torch.Tensor, reorder_index: torch.Tensor, BN: torch.Tensor, BS: torch.Tensor, BO: torch.Tensor,
                    SFBN: torch.Tensor, SFBS: torch.Tensor, SFBO: torch.Tensor, KN: int, KS: int, KO: int,
                    w_tiled: bool = False) -> torch.Tensor:
    return abi.fused_linear(X, reorder_index, BN, BS, BO, SFBN, SFBS, SFBO, KN, KS, KO, w_tiled=w_tiled)


@fused_linear_op.register_fake
def _(X, reorder_index, BN, BS, BO, SFBN, SFBS, SFBO, KN, KS, KO, w_tiled=False):
    n = BN.shape[0] if KN else (BS.shape[0] if KS else BO.shape[0])
    return torch.empty((X.shape[0], n), dtype=torch.bfloat16, device=X.device)


@torch.library.custom_op("mixedgemm_amd::fused_norm_linear", mutates_args=())
def fused_norm_linear_op(X: torch.Tensor, norm_weight: torch.Tensor, eps: float, reorder_index: torch.Tensor,
                         BN: torch.Tensor, BS: torch.Tensor, BO: torch.Tensor, SFBN: torch.Tensor, SFBS: torch.Tensor,
                         SFBO: torch.Tensor, KN: int, KS: int, KO: int, w_tiled: bool = False) -> torch.Tensor:
    return abi.fused_linear(X, reorder_index, BN, BS, BO, SFBN, SFBS, SFBO, KN, KS, KO, w_tiled=w_tiled,
                            norm_weight=norm_weight, eps=eps)


@fused_norm_linear_op.register_fake
def _(X, norm_weight, eps, reorder_index, BN, BS, BO, SFBN, SFBS, SFBO, KN, KS, KO, w_tiled=False):
    n = BN.shape[0] if KN else (BS.shape[0] if KS else BO.shape[0])
    return torch.empty((X.shape[0], n), dtype=torch.bfloat16, device=X.device)


@torch.library.custom_op("mixedgemm_amd::calibrate_reorder_index", mutates_args=())
def calibrate_reorder_index_op(X: torch.Tensor) -> torch.Tensor:
    return abi.calibrate_reorder_index(X)


@calibrate_reorder_index_op.register_fake
def _(X):
    return torch.empty((X.shape[1],), dtype=torch.int16, device=X.device)


# ------------------------------------------------------------------ the layer
class MixedLinear(torch.nn.Module):
    """y = quantize(x[..., reorder_index]) @ Wq^T (+ bias): the reference's three calls
    (main.py:35-37) with the weights quantized once.  Inference only.  With norm_weight (bf16 [K]) the
    input first passes through an RMSNorm, computed inside the quantizer's pass over the rows; the
    reorder index must then have been calibrated on normalised activations."""

    def __init__(self, packed: PackedWeights, bias: torch.Tensor | None = None,
                 norm_weight: torch.Tensor | None = None, eps: float = 1e-5):
        super().__init__()
        self.eps = float(eps)
        packed.validate()
        self.split = packed.split
        self.tiled = packed.tiled
        self.in_features, self.out_features = packed.in_features, packed.out_features
        for name in _SECTIONS:
            self.register_buffer(name, getattr(packed, name))
        self.register_buffer("bias", bias)
        self.register_buffer("norm_weight", norm_weight)

    @classmethod
    def from_float(cls, weight: torch.Tensor, calibration_x: torch.Tensor | None = None,
                   reorder_index: torch.Tensor | None = None, split=None, bias=None, tile=True) -> "MixedLinear":
        """weight bf16 [N, K] on the GPU; the reorder index comes from a calibration sample
        [tokens, K] unless it is given."""
        if reorder_index is None:
            if calibration_x is None:
                raise ValueError("give a calibration sample or a reorder index")
            reorder_index = torch.ops.mixedgemm_amd.calibrate_reorder_index(
                calibration_x.reshape(-1, calibration_x.shape[-1]).contiguous())
        return cls(PackedWeights.from_float(weight, reorder_index, split, tile), bias)

    def packed(self) -> PackedWeights:
        return PackedWeights(self.wn, self.ws, self.wo, self.sfwn, self.sfws, self.sfwo, self.reorder_index, self.split,
                             self.tiled, self.out_features if self.out_features != self.wn.shape[0] else 0)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.in_features)
        if x2.dtype != torch.bfloat16:
            x2 = x2.to(torch.bfloat16)
        if self.norm_weight is not None:
            y = torch.ops.mixedgemm_amd.fused_norm_linear(x2.contiguous(), self.norm_weight, self.eps, self.reorder_index,
                                                          self.wn, self.ws, self.wo, self.sfwn, self.sfws, self.sfwo,
                                                          *self.split, self.tiled)
        else:
            y = torch.ops.mixedgemm_amd.fused_linear(x2.contiguous(), self.reorder_index, self.wn, self.ws, self.wo,
                                                     self.sfwn, self.sfws, self.sfwo, *self.split, self.tiled)
        if y.shape[1] != self.out_features:
            y = y[:, :self.out_features]       # the padding rows of the weights
        if self.bias is not None:
            y = y + self.bias
        return y.reshape(*lead, self.out_features)

"""ctypes binding of the C-ABI in include/mixedgemm_abi.h.

Device memory and streams come from torch; every compute call goes into
libmixedgemm_hip.so.  There is no fallback: if the library has not been built
the first call raises.
"""
from __future__ import annotations

import ctypes
import os

import torch

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libmixedgemm_hip.so")

MG_OPERAND_A = 0
MG_OPERAND_B = 1
MG_FLAG_W_TILED = 1

SYMBOLS = (
    "mg_reorder_quantize_x", "mg_reorder_quantize_w", "mg_mixed_gemm", "mg_mixed_gemm_ex", "mg_padded_rows", "mg_tile_weights",
    "mg_weights_tileable", "mg_fused_linear_ex", "mg_rmsnorm_reorder_quantize_x", "mg_fused_norm_linear",
    "mg_fused_linear",
    "mg_fused_workspace_bytes", "mg_sf_bytes", "mg_sf_offset", "mg_device_synchronize", "mg_status_string",
    "mg_calibrate_reorder_index", "mg_calibrate_workspace_bytes", "mg_check_reorder_index", "mg_check_reorder_index_host",
    "mg_fused_linear_static",
)
MG_STATIC_SCRATCH_BYTES = 20 << 20

_lib = None


class MixedGemmError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MixedGemmError(
                f"{LIB_PATH} is missing: build it with `python -m mixedgemm_amd.build` "
                "(there is no non-HIP fallback)")
        L = ctypes.CDLL(LIB_PATH)
        p, i, z = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
        for name in ("mg_reorder_quantize_x", "mg_reorder_quantize_w"):
            fn = getattr(L, name)
            fn.restype, fn.argtypes = i, [p, p, i, i, i, i, i, p, p, p, p, p, p, p]
        L.mg_mixed_gemm.restype, L.mg_mixed_gemm.argtypes = i, [p] * 12 + [i] * 5 + [p, p]
        u = ctypes.c_uint
        L.mg_mixed_gemm_ex.restype, L.mg_mixed_gemm_ex.argtypes = i, [p] * 12 + [i] * 6 + [u, p, p]
        L.mg_tile_weights.restype, L.mg_tile_weights.argtypes = i, [p, p, i, i, p]
        L.mg_weights_tileable.restype, L.mg_weights_tileable.argtypes = i, [i, i, i, i]
        f = ctypes.c_float
        L.mg_rmsnorm_reorder_quantize_x.restype = i
        L.mg_rmsnorm_reorder_quantize_x.argtypes = [p, p, f, p, i, i, i, i, i, p, p, p, p, p, p, p]
        L.mg_fused_norm_linear.restype = i
        L.mg_fused_norm_linear.argtypes = [p, p, f, p] + [p] * 6 + [i] * 5 + [u, p, p, z, p]
        L.mg_fused_linear_ex.restype = i
        L.mg_fused_linear_ex.argtypes = [p] * 8 + [i] * 5 + [u, p, p, z, p]
        L.mg_padded_rows.restype, L.mg_padded_rows.argtypes = i, [i]
        L.mg_fused_linear.restype = i
        L.mg_fused_linear.argtypes = [p] * 8 + [i] * 5 + [p, p, z, p]
        L.mg_fused_workspace_bytes.restype, L.mg_fused_workspace_bytes.argtypes = z, [i, i, i, i]
        L.mg_sf_bytes.restype, L.mg_sf_bytes.argtypes = z, [i, i, i]
        L.mg_sf_offset.restype, L.mg_sf_offset.argtypes = z, [i, i, i]
        L.mg_device_synchronize.restype, L.mg_device_synchronize.argtypes = i, []
        L.mg_calibrate_reorder_index.restype, L.mg_calibrate_reorder_index.argtypes = i, [p, i, i, p, p, z, p]
        L.mg_calibrate_workspace_bytes.restype, L.mg_calibrate_workspace_bytes.argtypes = z, [i]
        L.mg_check_reorder_index.restype, L.mg_check_reorder_index.argtypes = i, [p, i, p]
        L.mg_check_reorder_index_host.restype, L.mg_check_reorder_index_host.argtypes = i, [p, i]
        L.mg_fused_linear_static.restype = i
        L.mg_fused_linear_static.argtypes = [p] * 8 + [i] * 5 + [u, p, p]
        L.mg_status_string.restype, L.mg_status_string.argtypes = ctypes.c_char_p, [i]
        _lib = L
    return _lib


def status_string(status: int) -> str:
    return lib().mg_status_string(int(status)).decode()


def check(status: int, what: str) -> None:
    if status != 0:
        raise MixedGemmError(f"{what} failed: {status_string(status)} (status {status})")


def sf_bytes(rows: int, kseg: int, operand: int) -> int:
    return int(lib().mg_sf_bytes(rows, kseg, operand))


def sf_offset(row: int, kb: int, kseg: int) -> int:
    return int(lib().mg_sf_offset(row, kb, kseg))


def fused_workspace_bytes(m: int, kn: int, ks: int, ko: int) -> int:
    return int(lib().mg_fused_workspace_bytes(m, kn, ks, ko))


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() else ctypes.c_void_p(0)


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _require(t: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    if t.dtype != dtype:
        raise MixedGemmError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_cuda:
        raise MixedGemmError(f"{name}: expected a GPU tensor")
    if not t.is_contiguous():
        raise MixedGemmError(f"{name}: expected a contiguous tensor")


def padded_rows(m: int) -> int:
    return int(lib().mg_padded_rows(m))


def _rows_view(alloc_rows, rows, cols, **kw):
    """uint8 [rows, cols] at the start of storage with room for alloc_rows rows."""
    return torch.empty((alloc_rows, cols), **kw)[:rows]


def _check_out(out, shape, dtype, name):
    """A caller-provided output must be what the call would have allocated."""
    _require(out, dtype, name)
    if tuple(out.shape) != tuple(shape):
        raise MixedGemmError(f"{name}: expected shape {tuple(shape)}, got {tuple(out.shape)}")


def _check_quant_out(out, rows, kn, ks, ko, operand):
    if len(out) != 6:
        raise MixedGemmError("out: expected six tensors (codes x3, scales x3)")
    w = operand == MG_OPERAND_B
    shapes = ((rows, kn // 2), (rows, ks // 2 if w else ks // 4 * 3), (rows, ko // 2 if w else ko))
    for t, shape, name in zip(out[:3], shapes, ("qn", "qs", "qo")):
        _check_out(t, shape, torch.uint8, name)
    for t, kseg, name in zip(out[3:], (kn, ks, ko), ("sfn", "sfs", "sfo")):
        _require(t, torch.uint8, name)
        if t.numel() < sf_bytes(rows, kseg, operand):
            raise MixedGemmError(f"{name}: {t.numel()} bytes, need {sf_bytes(rows, kseg, operand)}")


def alloc_quant_outputs(rows, kn, ks, ko, operand, device):
    """The six output tensors of a reorder-quantize call (codes x3, scales x3), with the
    reference's shapes.  For activations the storage behind them has room for whole 256-row
    tiles, which lets matmul() run a ragged token count on the whole-tile kernel."""
    w = operand == MG_OPERAND_B
    u8 = dict(dtype=torch.uint8, device=device)
    r = rows if w else padded_rows(rows)

    def sf(kseg):
        return torch.empty(max(sf_bytes(r, kseg, operand), sf_bytes(rows, kseg, operand)), **u8)[:sf_bytes(rows, kseg, operand)]

    return (_rows_view(r, rows, kn // 2, **u8),
            _rows_view(r, rows, ks // 2 if w else ks // 4 * 3, **u8),
            _rows_view(r, rows, ko // 2 if w else ko, **u8),
            sf(kn), sf(ks), sf(ko))


def _capacity(t: torch.Tensor) -> int:
    """Bytes readable from t's first element to the end of its storage."""
    return t.untyped_storage().nbytes() - t.storage_offset() * t.element_size()


def _reorder_quantize(fn_name, operand, t, idx, kn, ks, ko, out=None):
    _require(t, torch.bfloat16, "input")
    _require(idx, torch.int16, "reorder_index")
    rows, k = t.shape
    if idx.numel() != k:
        raise MixedGemmError(f"reorder_index has {idx.numel()} entries, input has {k} channels")
    if out is None:
        out = alloc_quant_outputs(rows, kn, ks, ko, operand, t.device)
    else:
        _check_quant_out(out, rows, kn, ks, ko, operand)
    qn, qs, qo, sfn, sfs, sfo = out
    status = getattr(lib(), fn_name)(_ptr(t), _ptr(idx), rows, k, kn, ks, ko,
                                     _ptr(qn), _ptr(qs), _ptr(qo), _ptr(sfn), _ptr(sfs), _ptr(sfo), _stream(t))
    check(status, fn_name)
    return qn, qs, qo, sfn, sfs, sfo


def reorder_quantize_x(x, reorder_index, kn, ks, ko, out=None):
    """(XN, XS, XO, SFXN, SFXS, SFXO); asynchronous on torch's current stream.
    `out` may carry six preallocated tensors (see alloc_quant_outputs)."""
    return _reorder_quantize("mg_reorder_quantize_x", MG_OPERAND_A, x, reorder_index, kn, ks, ko, out)


def rmsnorm_reorder_quantize_x(x, norm_weight, eps, reorder_index, kn, ks, ko, out=None):
    """reorder_quantize_x of RMSNorm(x) with bf16 weight norm_weight[K], in one pass over the rows
    (the arithmetic is spelled out at mg_rmsnorm_reorder_quantize_x in the header)."""
    _require(x, torch.bfloat16, "input")
    _require(norm_weight, torch.bfloat16, "norm_weight")
    _require(reorder_index, torch.int16, "reorder_index")
    rows, k = x.shape
    if reorder_index.numel() != k or norm_weight.numel() != k:
        raise MixedGemmError(f"reorder_index / norm_weight must have {k} entries")
    if out is None:
        out = alloc_quant_outputs(rows, kn, ks, ko, MG_OPERAND_A, x.device)
    else:
        _check_quant_out(out, rows, kn, ks, ko, MG_OPERAND_A)
    qn, qs, qo, sfn, sfs, sfo = out
    check(lib().mg_rmsnorm_reorder_quantize_x(_ptr(x), _ptr(norm_weight), float(eps), _ptr(reorder_index), rows, k, kn, ks,
                                              ko, _ptr(qn), _ptr(qs), _ptr(qo), _ptr(sfn), _ptr(sfs), _ptr(sfo),
                                              _stream(x)), "mg_rmsnorm_reorder_quantize_x")
    return qn, qs, qo, sfn, sfs, sfo


def reorder_quantize_w(w, reorder_index, kn, ks, ko, out=None):
    """(WN, WS, WO, SFWN, SFWS, SFWO); asynchronous on torch's current stream."""
    return _reorder_quantize("mg_reorder_quantize_w", MG_OPERAND_B, w, reorder_index, kn, ks, ko, out)


def matmul(an, bn, as_, bs, ao, bo, sfan, sfbn, sfas, sfbs, sfao, sfbo, out=None, w_tiled=False):
    """bf16 [M, N]; shapes are recovered from the packed operands.  w_tiled: bn, bs, bo are in the
    tile-major order of tile_weights()."""
    for name, t in (("AN", an), ("BN", bn), ("AS", as_), ("BS", bs), ("AO", ao), ("BO", bo),
                    ("SFAN", sfan), ("SFBN", sfbn), ("SFAS", sfas), ("SFBS", sfbs), ("SFAO", sfao), ("SFBO", sfbo)):
        _require(t, torch.uint8, name)
    m, n = an.shape[0], bn.shape[0]
    kn, ks, ko = an.shape[1] * 2, as_.shape[1] * 4 // 3, ao.shape[1]
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=an.device)
    else:
        _check_out(out, (m, n), torch.bfloat16, "out")
    if bs.shape[0] != n or bo.shape[0] != n or as_.shape[0] != m or ao.shape[0] != m:
        raise MixedGemmError("the three segments of an operand must have the same number of rows")
    if bn.shape[1] * 2 != kn or bs.shape[1] * 2 != ks or bo.shape[1] * 2 != ko:
        raise MixedGemmError("activation and weight segments disagree on KN / KS / KO")
    for t in (bn, as_, bs, ao, bo, sfan, sfbn, sfas, sfbs, sfao, sfbo, out):
        if t.device != an.device:
            raise MixedGemmError("all operands must be on the same GPU")
    for name, t, rows, kseg, operand in (("SFAN", sfan, m, kn, MG_OPERAND_A), ("SFAS", sfas, m, ks, MG_OPERAND_A),
                                         ("SFAO", sfao, m, ko, MG_OPERAND_A), ("SFBN", sfbn, n, kn, MG_OPERAND_B),
                                         ("SFBS", sfbs, n, ks, MG_OPERAND_B), ("SFBO", sfbo, n, ko, MG_OPERAND_B)):
        if t.numel() < sf_bytes(rows, kseg, operand):
            raise MixedGemmError(f"{name}: {t.numel()} bytes, need {sf_bytes(rows, kseg, operand)}")
    # rows the activation buffers are readable for: whole tiles if every storage has the room
    r = padded_rows(m)
    roomy = all(_capacity(t) >= r * t.shape[1] for t in (an, as_, ao)) and all(
        _capacity(t) >= sf_bytes(r, kseg, MG_OPERAND_A) for t, kseg in ((sfan, kn), (sfas, ks), (sfao, ko)) if kseg)
    status = lib().mg_mixed_gemm_ex(_ptr(an), _ptr(bn), _ptr(as_), _ptr(bs), _ptr(ao), _ptr(bo),
                                    _ptr(sfan), _ptr(sfbn), _ptr(sfas), _ptr(sfbs), _ptr(sfao), _ptr(sfbo),
                                    m, r if roomy else m, n, kn, ks, ko, MG_FLAG_W_TILED if w_tiled else 0,
                                    _ptr(out), _stream(an))
    check(status, "mg_mixed_gemm")
    return out


def _check_weights(x, bn, bs, bo, sfbn, sfbs, sfbo, kn, ks, ko):
    """The six weight tensors of a fused call: uint8, contiguous, on x's GPU, [N, kseg / 2] codes and scale
    buffers of at least the size the GEMM reads.  Returns N."""
    for name, t in (("BN", bn), ("BS", bs), ("BO", bo), ("SFBN", sfbn), ("SFBS", sfbs), ("SFBO", sfbo)):
        _require(t, torch.uint8, name)
        if t.device != x.device:
            raise MixedGemmError(f"{name}: on {t.device}, X is on {x.device}")
    for name, t in (("BN", bn), ("BS", bs), ("BO", bo)):
        if t.dim() != 2:
            raise MixedGemmError(f"{name}: expected a 2-D tensor")
    n = bn.shape[0]
    for name, t, kseg in (("BN", bn, kn), ("BS", bs, ks), ("BO", bo, ko)):
        if tuple(t.shape) != (n, kseg // 2):
            raise MixedGemmError(f"{name}: expected shape {(n, kseg // 2)}, got {tuple(t.shape)}")
    for name, t, kseg in (("SFBN", sfbn, kn), ("SFBS", sfbs, ks), ("SFBO", sfbo, ko)):
        if t.numel() < sf_bytes(n, kseg, MG_OPERAND_B):
            raise MixedGemmError(f"{name}: {t.numel()} bytes, need {sf_bytes(n, kseg, MG_OPERAND_B)}")
    return n


def _check_fused_inputs(x, reorder_index, kn, ks, ko):
    _require(x, torch.bfloat16, "X")
    _require(reorder_index, torch.int16, "reorder_index")
    if x.dim() != 2:
        raise MixedGemmError("X: expected a 2-D tensor")
    if min(kn, ks, ko) < 0 or (kn | ks | ko) % 32:
        raise MixedGemmError("KN, KS, KO must be non-negative multiples of 32")
    if x.shape[1] != kn + ks + ko or reorder_index.numel() != x.shape[1]:
        raise MixedGemmError(f"X has {x.shape[1]} channels, the split sums to {kn + ks + ko}, the index has {reorder_index.numel()}")
    if reorder_index.device != x.device:
        raise MixedGemmError(f"reorder_index: on {reorder_index.device}, X is on {x.device}")


def fused_linear(x, reorder_index, bn, bs, bo, sfbn, sfbs, sfbo, kn, ks, ko, workspace=None, out=None, w_tiled=False,
                 norm_weight=None, eps=0.0):
    """Activation reorder-quantize + mixed GEMM on one stream; returns bf16 [M, N].  With norm_weight
    (bf16 [K]) the activations pass through an RMSNorm first, inside the quantizer's row pass."""
    _check_fused_inputs(x, reorder_index, kn, ks, ko)
    m = x.shape[0]
    n = _check_weights(x, bn, bs, bo, sfbn, sfbs, sfbo, kn, ks, ko)
    need = fused_workspace_bytes(m, kn, ks, ko)
    if workspace is None:
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    else:
        _check_out(out, (m, n), torch.bfloat16, "out")
    _require(workspace, torch.uint8, "workspace")
    if workspace.numel() < need or workspace.device != x.device or out.device != x.device:
        raise MixedGemmError(f"workspace: need {need} uint8 on X's GPU (and `out` there too)")
    if norm_weight is not None:
        _require(norm_weight, torch.bfloat16, "norm_weight")
        if norm_weight.numel() != x.shape[1] or norm_weight.device != x.device:
            raise MixedGemmError(f"norm_weight must have {x.shape[1]} entries on X's GPU")
    status = lib().mg_fused_norm_linear(_ptr(x), _ptr(norm_weight), float(eps), _ptr(reorder_index), _ptr(bn), _ptr(bs),
                                        _ptr(bo), _ptr(sfbn), _ptr(sfbs), _ptr(sfbo), m, n, kn, ks, ko,
                                        MG_FLAG_W_TILED if w_tiled else 0,
                                        _ptr(out), _ptr(workspace), workspace.numel(), _stream(x))
    check(status, "mg_fused_norm_linear")
    return out


def fused_linear_static(x, reorder_index, bn, bs, bo, sfbn, sfbs, sfbo, kn, ks, ko, out, w_tiled=False):
    """fused_linear through the library's own static scratch memory: the call allocates nothing, so `out`
    (bf16 [M, N]) is the caller's.  Problems whose quantized activations exceed MG_STATIC_SCRATCH_BYTES are
    rejected; calls on one GPU must not overlap (they share the scratch memory)."""
    _check_fused_inputs(x, reorder_index, kn, ks, ko)
    m = x.shape[0]
    n = _check_weights(x, bn, bs, bo, sfbn, sfbs, sfbo, kn, ks, ko)
    _check_out(out, (m, n), torch.bfloat16, "out")
    if out.device != x.device:
        raise MixedGemmError("out must be on X's GPU")
    status = lib().mg_fused_linear_static(_ptr(x), _ptr(reorder_index), _ptr(bn), _ptr(bs), _ptr(bo), _ptr(sfbn),
                                          _ptr(sfbs), _ptr(sfbo), m, n, kn, ks, ko, MG_FLAG_W_TILED if w_tiled else 0,
                                          _ptr(out), _stream(x))
    check(status, "mg_fused_linear_static")
    return out


def check_reorder_index(reorder_index, k=None) -> None:
    """Raises MixedGemmError unless every entry of the int16 index lies in [0, K).  Blocks for a GPU tensor."""
    if reorder_index.dtype != torch.int16 or not reorder_index.is_contiguous():
        raise MixedGemmError("reorder_index: expected a contiguous int16 tensor")
    k = reorder_index.numel() if k is None else int(k)
    if reorder_index.numel() != k:
        raise MixedGemmError(f"reorder_index has {reorder_index.numel()} entries, expected {k}")
    if reorder_index.is_cuda:
        status = lib().mg_check_reorder_index(_ptr(reorder_index), k, _stream(reorder_index))
    else:
        status = lib().mg_check_reorder_index_host(ctypes.c_void_p(reorder_index.data_ptr()), k)
    check(status, "mg_check_reorder_index")


def weights_tileable(n: int, kn: int, ks: int, ko: int) -> bool:
    return bool(lib().mg_weights_tileable(n, kn, ks, ko))


def tile_weights(wn, ws, wo):
    """The three weight code tensors of reorder_quantize_w, rewritten into the tile-major order the
    prefill kernel copies fastest (same shapes and sizes; pass w_tiled=True to matmul / fused_linear)."""
    out = []
    for t in (wn, ws, wo):
        _require(t, torch.uint8, "weights")
        dst = torch.empty_like(t)
        check(lib().mg_tile_weights(_ptr(t), _ptr(dst), t.shape[0], t.shape[1] * 2, _stream(t)), "mg_tile_weights")
        out.append(dst)
    return tuple(out)


def calibrate_reorder_index(x, out=None, workspace=None):
    """Reorder index of a bf16 activation sample x[M, K]: channels by ascending max |x| over the
    rows, ties by channel number, int16 (main.py:31-33 of the reference, there as torch calls)."""
    _require(x, torch.bfloat16, "x")
    if x.dim() != 2:
        raise MixedGemmError(f"x: expected a 2-D tensor [rows, channels], got {x.dim()} dimensions")
    m, k = x.shape
    need = int(lib().mg_calibrate_workspace_bytes(k))
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    if out is None:
        out = torch.empty(k, dtype=torch.int16, device=x.device)
    else:
        _check_out(out, (k,), torch.int16, "out")
    if workspace.numel() < need or not workspace.is_cuda:
        raise MixedGemmError(f"workspace: need {need} bytes on the GPU")
    check(lib().mg_calibrate_reorder_index(_ptr(x), m, k, _ptr(out), _ptr(workspace), workspace.numel(),
                                           _stream(x)), "mg_calibrate_reorder_index")
    return out


def device_synchronize() -> None:
    check(lib().mg_device_synchronize(), "mg_device_synchronize")

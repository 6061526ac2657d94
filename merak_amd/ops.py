"""Tensor-level wrappers over the C ABI: shape/dtype/device checks, output
allocation through PyTorch's caching allocator, and the current HIP stream.

PyTorch is plumbing here (device memory and streams); every FLOP and every
byte moved happens inside ``libmerak_tp_gfx950.so``.  CPU tensors are rejected:
there is no fallback path.
"""
from __future__ import annotations

import threading
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import (EPI_BIAS, EPI_BIAS_GELU, EPI_GELU, EPI_NONE, EPI_SWIGLU,
                   MTP_BF16, MTP_F16, MTP_F32)

_DTYPES = {torch.float32: MTP_F32, torch.bfloat16: MTP_BF16, torch.float16: MTP_F16}
_arch_ok = {}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"merak_amd kernels take float32, bfloat16 or float16 tensors, got {t.dtype}") from None


def _require_gpu(*ts: torch.Tensor) -> torch.device:
    dev = None
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "merak_amd kernels run on an MI355X (gfx950) device only; got a tensor on "
                f"{t.device}. There is no CPU fallback.")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    if idx not in _arch_ok:
        with torch.cuda.device(idx):
            arch = _lib.device_arch()
        if arch != "gfx950":
            raise RuntimeError(f"merak_amd kernels are built for gfx950 only; device {idx} is {arch}")
        _arch_ok[idx] = True
    return dev


def _stream(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _contig(t: torch.Tensor) -> torch.Tensor:
    return t if t.is_contiguous() else t.contiguous()


# --------------------------------------------------------------------------- linear
_linear_ws_cache = {}
_linear_ws_lock = threading.Lock()   # forward runs on the caller's thread, backward on autograd's worker thread


def linear_workspace(dev: torch.device, nbytes: Optional[int] = None) -> torch.Tensor:
    """Scratch of the linear products for the current stream of `dev` (16-bit: stream-K, tiles whose k range
    several workgroups share meet there; fp32: the slices of a product that is cut along k), at least `nbytes`
    long (default: the 16-bit path's full size).  One buffer per (device, stream), allocated when a product first
    asks for scratch and grown when a later one asks for more: launches on one stream are ordered, so they may
    share it.  ``release_workspaces()`` drops them all."""
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    key = (idx, torch.cuda.current_stream(dev).cuda_stream)
    if nbytes is None:
        nbytes = _lib.lib().mtp_linear_workspace_bytes()
    with _linear_ws_lock:
        ws = _linear_ws_cache.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(int(nbytes), dtype=torch.uint8, device=dev)
            _linear_ws_cache[key] = ws
    return ws


def release_workspaces() -> None:
    """Forget the cached scratch buffers of the linear products (they are allocated again on demand)."""
    with _linear_ws_lock:
        _linear_ws_cache.clear()


def _ws_args(kind: int, M: int, N: int, K: int, t: torch.Tensor, dev: torch.device):
    """(pointer, bytes) of the scratch for product `kind` (0 forward, 1 input gradient, 2 weight gradient, 3 both
    gradients) of a layer with M tokens, N output and K input features on tensors like t; (None, 0) for the shapes
    that never use scratch, which then allocate nothing."""
    need = _lib.lib().mtp_linear_workspace_need(kind, M, N, K, _dt(t))
    if need <= 0:
        return None, 0
    ws = linear_workspace(dev, need)
    return ws.data_ptr(), ws.numel()


def linear_fwd(x2d: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], epilogue: int = EPI_NONE,
               want_pre: bool = True, lead: Optional[Tuple[int, ...]] = None
               ) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """(y, act) = epilogue(x2d @ w.T + bias).  x2d [M,K], w [N,K] contiguous, same dtype.  lead: leading
    dimensions (product M) to allocate the outputs with, so that a caller whose input was [*lead, K] gets
    [*lead, N] tensors that own their storage instead of views of [M, N] ones."""
    dev = _require_gpu(x2d, w, bias)
    if x2d.dim() != 2 or w.dim() != 2:
        raise ValueError(f"linear_fwd: x must be [M, K] and weight [N, K], got {tuple(x2d.shape)} and {tuple(w.shape)}")
    M, K = x2d.shape
    N, K2 = w.shape
    if K != K2:
        raise ValueError(f"linear_fwd: x is [*, {K}] but weight is [{N}, {K2}]")
    if w.dtype != x2d.dtype or (bias is not None and bias.dtype != x2d.dtype):
        raise TypeError("linear_fwd: x, weight and bias must share one dtype")
    if bias is not None and (bias.numel() != N or not bias.is_contiguous()):
        raise ValueError(f"linear_fwd: bias must be a contiguous [{N}] tensor, got {tuple(bias.shape)}")
    if epilogue == EPI_SWIGLU and N % 2:
        raise ValueError(f"linear_fwd: SwiGLU needs an even number of weight rows, got {N}")
    x2d, w = _contig(x2d), _contig(w)
    has_act = epilogue in (EPI_BIAS_GELU, EPI_SWIGLU, EPI_GELU)
    rows = (M,) if lead is None else tuple(lead)
    if lead is not None:
        prod = 1
        for d in rows:
            prod *= d
        if prod != M:
            raise ValueError(f"linear_fwd: leading dimensions {rows} do not hold {M} rows")
    y = torch.empty(rows + (N,), dtype=x2d.dtype, device=dev) if (want_pre or not has_act) else None
    act = None
    if has_act:
        act = torch.empty(rows + (N // 2 if epilogue == EPI_SWIGLU else N,), dtype=x2d.dtype, device=dev)
    with torch.cuda.device(dev):
        wsp, wsb = _ws_args(0, M, N, K, x2d, dev)
        rc = _lib.lib().mtp_linear_fwd_ws(_p(x2d), _p(w), _p(bias), _p(y), _p(act), wsp, wsb, M, N, K, _dt(x2d),
                                          epilogue, _stream(dev))
        if rc == -2 and y is None:
            # shapes served by the general kernel need the pre-activation buffer for SwiGLU
            y = torch.empty((M, N), dtype=x2d.dtype, device=dev)
            rc = _lib.lib().mtp_linear_fwd_ws(_p(x2d), _p(w), _p(bias), _p(y), _p(act), wsp, wsb, M, N, K, _dt(x2d),
                                              epilogue, _stream(dev))
            y = None
        _lib.check(rc, "mtp_linear_fwd")
    return y, act


def linear_dgrad(dy2d: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    dev = _require_gpu(dy2d, w)
    if dy2d.dim() != 2 or w.dim() != 2:
        raise ValueError(f"linear_dgrad: dy must be [M, N] and weight [N, K], got {tuple(dy2d.shape)} and {tuple(w.shape)}")
    M, N = dy2d.shape
    N2, K = w.shape
    if N != N2 or dy2d.dtype != w.dtype:
        raise ValueError("linear_dgrad: dy/weight mismatch")
    dy2d, w = _contig(dy2d), _contig(w)
    dx = torch.empty((M, K), dtype=dy2d.dtype, device=dev)
    with torch.cuda.device(dev):
        wsp, wsb = _ws_args(1, M, N, K, dy2d, dev)
        _lib.check(_lib.lib().mtp_linear_dgrad_ws(_p(dy2d), _p(w), _p(dx), wsp, wsb, M, N, K, _dt(dy2d), _stream(dev)),
                   "mtp_linear_dgrad")
    return dx


def linear_wgrad(dy2d: torch.Tensor, x2d: torch.Tensor, want_db: bool, out_dtype: Optional[torch.dtype] = None,
                 dw: Optional[torch.Tensor] = None, db: Optional[torch.Tensor] = None,
                 accumulate: bool = False) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    dev = _require_gpu(dy2d, x2d, dw, db)
    if dy2d.dim() != 2 or x2d.dim() != 2:
        raise ValueError(f"linear_wgrad: dy must be [M, N] and x [M, K], got {tuple(dy2d.shape)} and {tuple(x2d.shape)}")
    M, N = dy2d.shape
    M2, K = x2d.shape
    if M != M2 or dy2d.dtype != x2d.dtype:
        raise ValueError("linear_wgrad: dy/x mismatch")
    dy2d, x2d = _contig(dy2d), _contig(x2d)
    out_dtype = out_dtype or (dw.dtype if dw is not None else dy2d.dtype)
    if dw is None:
        if accumulate:
            raise ValueError("linear_wgrad: accumulate needs an existing dw")
        dw = torch.empty((N, K), dtype=out_dtype, device=dev)
    if want_db and db is None:
        if accumulate:
            raise ValueError("linear_wgrad: accumulate needs an existing db")
        db = torch.empty((N,), dtype=out_dtype, device=dev)
    if dw.shape != (N, K) or not dw.is_contiguous() or dw.dtype != out_dtype:
        raise ValueError("linear_wgrad: dw must be a contiguous [N,K] tensor of the output dtype")
    if want_db and (db.numel() != N or not db.is_contiguous() or db.dtype != out_dtype):
        raise ValueError("linear_wgrad: db must be a contiguous [N] tensor of the output dtype")
    with torch.cuda.device(dev):
        wsp, wsb = _ws_args(2, M, N, K, dy2d, dev)
        _lib.check(_lib.lib().mtp_linear_wgrad_ws(_p(dy2d), _p(x2d), _p(dw), _p(db) if want_db else None, wsp, wsb, M, N,
                                                  K, _dt(dy2d), _DTYPES[out_dtype], int(accumulate), _stream(dev)),
                   "mtp_linear_wgrad")
    return dw, (db if want_db else None)


def linear_bwd(dy2d: torch.Tensor, x2d: torch.Tensor, w: torch.Tensor, want_db: bool,
               out_dtype: Optional[torch.dtype] = None, dw: Optional[torch.Tensor] = None,
               db: Optional[torch.Tensor] = None, accumulate: bool = False):
    """(dx, dw, db) = (dy w, dy^T x, sum of dy's rows): linear_dgrad and linear_wgrad of one layer as one call, and
    as one launch where the tiles of the two products together fill fewer rounds of workgroups than apart."""
    dev = _require_gpu(dy2d, x2d, w, dw, db)
    if dy2d.dim() != 2 or x2d.dim() != 2 or w.dim() != 2:
        raise ValueError("linear_bwd: dy [M, N], x [M, K] and weight [N, K] must be 2-d")
    M, N = dy2d.shape
    K = x2d.shape[1]
    if x2d.shape[0] != M or tuple(w.shape) != (N, K):
        raise ValueError(f"linear_bwd: shapes dy {tuple(dy2d.shape)}, x {tuple(x2d.shape)}, weight {tuple(w.shape)}")
    if not (dy2d.dtype == x2d.dtype == w.dtype):
        raise TypeError("linear_bwd: dy, x and weight must share a dtype")
    out_dtype = out_dtype or (dw.dtype if dw is not None else dy2d.dtype)
    if accumulate and dw is None:
        raise ValueError("linear_bwd: accumulate needs the gradient buffers")
    dy2d, x2d, w = _contig(dy2d), _contig(x2d), _contig(w)
    dx = torch.empty((M, K), dtype=dy2d.dtype, device=dev)
    if dw is None:
        dw = torch.empty((N, K), dtype=out_dtype, device=dev)
    if want_db and db is None:
        db = torch.empty((N,), dtype=out_dtype, device=dev)
    if tuple(dw.shape) != (N, K) or dw.dtype != out_dtype or not dw.is_contiguous():
        raise ValueError("linear_bwd: dw must be a contiguous [N, K] tensor of out_dtype")
    if want_db and (tuple(db.shape) != (N,) or db.dtype != out_dtype or not db.is_contiguous()):
        raise ValueError("linear_bwd: db must be a contiguous [N] tensor of out_dtype")
    with torch.cuda.device(dev):
        wsp, wsb = _ws_args(3, M, N, K, dy2d, dev)
        _lib.check(_lib.lib().mtp_linear_bwd_ws(_p(dy2d), _p(x2d), _p(w), _p(dx), _p(dw), _p(db) if want_db else None,
                                                wsp, wsb, M, N, K, _dt(dy2d), _DTYPES[out_dtype], int(accumulate),
                                                _stream(dev)), "mtp_linear_bwd")
    return dx, dw, (db if want_db else None)


def colsum(dy2d: torch.Tensor, db: torch.Tensor, accumulate: bool = False) -> torch.Tensor:
    """db (+)= dy2d.sum(0): the bias gradient alone, for a layer whose weight takes none."""
    dev = _require_gpu(dy2d, db)
    if dy2d.dim() != 2 or db.numel() != dy2d.shape[1] or not db.is_contiguous():
        raise ValueError(f"colsum: dy must be [M, N] and db a contiguous [N], got {tuple(dy2d.shape)} and {tuple(db.shape)}")
    if db.dtype not in (dy2d.dtype, torch.float32):
        raise TypeError("colsum: db must have dy's dtype or float32")
    dy2d = _contig(dy2d)
    M, N = dy2d.shape
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_linear_bias_grad(_p(dy2d), _p(db), M, N, _dt(dy2d), _DTYPES[db.dtype], int(accumulate),
                                                   _stream(dev)), "mtp_linear_bias_grad")
    return db


def activation_bwd(dact: torch.Tensor, y: torch.Tensor, epilogue: int) -> torch.Tensor:
    dev = _require_gpu(dact, y)
    if y.dim() != 2 or dact.dim() != 2 or dact.dtype != y.dtype:
        raise ValueError("activation_bwd: dact and y must be 2-D tensors of one dtype")
    M, N = y.shape
    if tuple(dact.shape) != (M, N // 2 if epilogue == EPI_SWIGLU else N):
        raise ValueError(f"activation_bwd: dact {tuple(dact.shape)} does not match y {tuple(y.shape)} for epilogue {epilogue}")
    dact, y = _contig(dact), _contig(y)
    dy = torch.empty_like(y)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_activation_bwd(_p(dact), _p(y), _p(dy), M, N, _dt(y), epilogue, _stream(dev)),
                   "mtp_activation_bwd")
    return dy


# --------------------------------------------------------------------------- embedding
def embedding_gather(ids: torch.Tensor, table: torch.Tensor, vocab_start: int, vocab_end: int,
                     oob_count: Optional[torch.Tensor] = None) -> torch.Tensor:
    dev = _require_gpu(ids, table, oob_count)
    if ids.dtype != torch.int64:
        raise TypeError(f"embedding ids must be int64, got {ids.dtype}")
    if table.dim() != 2 or not table.is_contiguous():
        raise ValueError("embedding table must be a contiguous [rows, dim] tensor")
    if table.shape[0] != vocab_end - vocab_start:
        raise ValueError("embedding table rows do not match the vocab range")
    flat = _contig(ids).view(-1)
    out = torch.empty((flat.numel(), table.shape[1]), dtype=table.dtype, device=dev)
    row_bytes = table.shape[1] * table.element_size()
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_embedding_gather(_p(flat), _p(table), _p(out), flat.numel(), row_bytes, vocab_start,
                                                   vocab_end, _p(oob_count), _stream(dev)), "mtp_embedding_gather")
    return out.view(*ids.shape, table.shape[1])


def embedding_bwd(ids: torch.Tensor, dout: torch.Tensor, rows: int, vocab_start: int, vocab_end: int,
                  out: Optional[torch.Tensor] = None, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Dense gradient [rows, dim] of the lookup, reproducible bit for bit.

    ``out`` given: the gradient is added onto it (e.g. the tied LM head's weight gradient);
    otherwise a zero-filled table of ``dtype`` (default: dout's) is created."""
    dev = _require_gpu(ids, dout, out)
    flat = _contig(ids).view(-1)
    dim = dout.shape[-1]
    d2 = _contig(dout).view(-1, dim)
    if flat.dtype != torch.int64:
        raise TypeError(f"embedding ids must be int64, got {flat.dtype}")
    if d2.shape[0] != flat.numel():
        raise ValueError(f"embedding_bwd: {d2.shape[0]} gradient rows for {flat.numel()} ids")
    if rows != vocab_end - vocab_start:
        raise ValueError("embedding_bwd: table rows do not match the vocab range")
    if out is None:
        out = torch.zeros((rows, dim), dtype=dtype or d2.dtype, device=dev)
    elif tuple(out.shape) != (rows, dim) or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous [{rows}, {dim}] tensor")
    lib = _lib.lib()
    ws = torch.empty((max(int(lib.mtp_embedding_bwd_workspace_bytes(flat.numel(), dim)), 16),), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(lib.mtp_embedding_bwd(_p(flat), _p(d2), _p(out), _p(ws), ws.numel(), flat.numel(), dim, _dt(d2),
                                         _dt(out), vocab_start, vocab_end, _stream(dev)), "mtp_embedding_bwd")
    return out


# --------------------------------------------------------------------------- cross entropy
def vocab_ce_fwd(logits2d: torch.Tensor, target1d: torch.Tensor, vocab_start: int):
    """-> (loss, row_max, row_sumexp, pred), all fp32 [n_rows]."""
    dev = _require_gpu(logits2d, target1d)
    if target1d.dtype != torch.int64:
        raise TypeError(f"cross-entropy targets must be int64, got {target1d.dtype}")
    if not logits2d.is_contiguous():
        raise ValueError("vocab_parallel_cross_entropy needs contiguous logits")
    n, v = logits2d.shape
    if target1d.numel() != n:
        raise ValueError(f"target has {target1d.numel()} entries for {n} logits rows")
    target1d = _contig(target1d)
    out = torch.empty((4, n), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_vocab_ce_fwd(_p(logits2d), _p(target1d), _p(out[0]), _p(out[1]), _p(out[2]),
                                               _p(out[3]), n, v, vocab_start, _dt(logits2d), _stream(dev)),
                   "mtp_vocab_ce_fwd")
    return out[0], out[1], out[2], out[3]


def vocab_ce_bwd_(logits2d: torch.Tensor, target1d: torch.Tensor, row_max: Optional[torch.Tensor],
                  row_sumexp: Optional[torch.Tensor], grad_out: Optional[torch.Tensor], vocab_start: int) -> torch.Tensor:
    """In place: logits2d <- (softmax - onehot) * grad_out.  Returns logits2d.

    row_max = row_sumexp = None: logits2d already holds the softmax."""
    dev = _require_gpu(logits2d, target1d, row_max, row_sumexp, grad_out)
    if target1d.dtype != torch.int64:
        raise TypeError(f"cross-entropy targets must be int64, got {target1d.dtype}")
    if not logits2d.is_contiguous():
        raise ValueError("vocab_parallel_cross_entropy needs contiguous logits")
    n, v = logits2d.shape
    if target1d.numel() != n:
        raise ValueError(f"target has {target1d.numel()} entries for {n} logits rows")
    for name, t in (("row_max", row_max), ("row_sumexp", row_sumexp)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != n or not t.is_contiguous()):
            raise ValueError(f"vocab_ce_bwd_: {name} must be contiguous fp32 [{n}]")
    if grad_out is not None:
        grad_out = _contig(grad_out.to(torch.float32))
        if grad_out.numel() != n:
            raise ValueError(f"grad_out has {grad_out.numel()} entries for {n} logits rows")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_vocab_ce_bwd(_p(logits2d), _p(_contig(target1d)), _p(row_max), _p(row_sumexp),
                                               _p(grad_out), n, v, vocab_start, _dt(logits2d), _stream(dev)),
                   "mtp_vocab_ce_bwd")
    return logits2d


def vocab_ce_fused_max_vocab(dtype: torch.dtype) -> int:
    """Longest row the one-launch forward+backward kernel keeps in registers."""
    return int(_lib.lib().mtp_vocab_ce_fwd_bwd_max_vocab(_DTYPES[dtype]))


def vocab_ce_fwd_bwd_(logits2d: torch.Tensor, target1d: torch.Tensor, vocab_start: int,
                      grad_rows: Optional[torch.Tensor] = None, grad_scale: float = 1.0):
    """One launch: -> (loss, row_max, row_sumexp, pred) and, in place,
    logits2d <- (softmax - onehot) * grad_rows[i] * grad_scale."""
    dev = _require_gpu(logits2d, target1d, grad_rows)
    if target1d.dtype != torch.int64:
        raise TypeError(f"cross-entropy targets must be int64, got {target1d.dtype}")
    if not logits2d.is_contiguous():
        raise ValueError("vocab_parallel_cross_entropy needs contiguous logits")
    n, v = logits2d.shape
    if target1d.numel() != n:
        raise ValueError(f"target has {target1d.numel()} entries for {n} logits rows")
    if grad_rows is not None:
        grad_rows = _contig(grad_rows.to(torch.float32))
        if grad_rows.numel() != n:
            raise ValueError(f"grad_rows has {grad_rows.numel()} entries for {n} logits rows")
    target1d = _contig(target1d)
    out = torch.empty((4, n), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_vocab_ce_fwd_bwd(_p(logits2d), _p(target1d), _p(grad_rows), float(grad_scale),
                                                   _p(out[0]), _p(out[1]), _p(out[2]), _p(out[3]), n, v,
                                                   vocab_start, _dt(logits2d), _stream(dev)),
                   "mtp_vocab_ce_fwd_bwd")
    return out[0], out[1], out[2], out[3]


def vocab_ce_rescale_(grad2d: torch.Tensor, grad_rows: torch.Tensor, assumed: float) -> torch.Tensor:
    """In place: rows of grad2d whose grad_rows[i] differs from ``assumed`` are scaled by grad_rows[i]/assumed."""
    dev = _require_gpu(grad2d, grad_rows)
    n, v = grad2d.shape
    grad_rows = _contig(grad_rows.to(torch.float32))
    if grad_rows.numel() != n:
        raise ValueError(f"grad_rows has {grad_rows.numel()} entries for {n} rows")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_vocab_ce_rescale(_p(grad2d), _p(grad_rows), float(assumed), n, v, _dt(grad2d),
                                                   _stream(dev)), "mtp_vocab_ce_rescale")
    return grad2d


# --------------------------------------------------------------------------- decode
def gemv_workspace(B: int, N: int, K: int, epilogue: int, device) -> Optional[torch.Tensor]:
    """Zero-filled scratch for ``gemv(..., workspace=)`` or None when this shape runs without one.  One
    workspace serves any number of launches, of any shapes, that do not overlap: take the largest need (the
    counters every launch leaves zero sit in its first 8 KiB whatever the shape)."""
    need = int(_lib.lib().mtp_gemv_workspace_bytes(B, N, K, epilogue))
    return torch.zeros((need,), dtype=torch.uint8, device=device) if need else None


def _decode_dtype(what: str, *ts: torch.Tensor) -> torch.dtype:
    dt = ts[0].dtype
    if dt not in (torch.bfloat16, torch.float16) or any(t.dtype != dt for t in ts if t is not None):
        raise TypeError(f"{what} takes bfloat16 or float16 tensors of one dtype, got {[t.dtype for t in ts if t is not None]}")
    return dt


def _gemv_shapes(what: str, x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor]):
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise ValueError(f"{what}: x must be [B, K] and weight [N, K], got {tuple(x.shape)} and {tuple(w.shape)}")
    if bias is not None and (bias.numel() != w.shape[0] or not bias.is_contiguous()):
        raise ValueError(f"{what}: bias must be a contiguous [{w.shape[0]}] tensor, got {tuple(bias.shape)}")
    return x.shape[0], w.shape[0], x.shape[1]


def gemv(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, epilogue: int = EPI_NONE,
         workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    dev = _require_gpu(x, w, bias, workspace)
    dt = _decode_dtype("gemv", x, w, bias)
    B, N, K = _gemv_shapes("gemv", x, w, bias)
    x, w = _contig(x), _contig(w)
    y = torch.empty((B, N // 2 if epilogue == EPI_SWIGLU else N), dtype=dt, device=dev)
    wbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_gemv_ws(_p(x), _p(w), _p(bias), _p(y), _p(workspace), wbytes, B, N, K, epilogue,
                                          _DTYPES[dt], _stream(dev)), "mtp_gemv")
    return y


def gemv_pair(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, bias1: Optional[torch.Tensor] = None,
              bias2: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None):
    """``(x @ w1.T (+ bias1), swiglu(x @ w2.T (+ bias2)))``: two products over the same rows in one call (one
    launch above 16 rows, the two launches of ``gemv`` otherwise)."""
    dev = _require_gpu(x, w1, w2, bias1, bias2, workspace)
    dt = _decode_dtype("gemv_pair", x, w1, bias1)
    _decode_dtype("gemv_pair", x, w2, bias2)
    B, N1, K = _gemv_shapes("gemv_pair", x, w1, bias1)
    _, N2, K2 = _gemv_shapes("gemv_pair", x, w2, bias2)
    if K2 != K or N2 % 2:
        raise ValueError(f"gemv_pair: second weight must be [2 * I, {K}], got {tuple(w2.shape)}")
    x, w1, w2 = _contig(x), _contig(w1), _contig(w2)
    y1 = torch.empty((B, N1), dtype=dt, device=dev)
    act2 = torch.empty((B, N2 // 2), dtype=dt, device=dev)
    wbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_gemv_pair(_p(x), _p(w1), _p(bias1), _p(y1), N1, _p(w2), _p(bias2), _p(act2), N2,
                                            _p(workspace), wbytes, B, K, _DTYPES[dt], _stream(dev)), "mtp_gemv_pair")
    return y1, act2


def gemv_norm_fits(B: int, K: int) -> bool:
    """Whether ``gemv_fused`` can take the RMSNorm of a [B, K] input inside the product (B K <= 8 x 4096, K % 512 == 0, K <= 8192)."""
    return bool(_lib.lib().mtp_gemv_norm_fits(B, K))


def gemv_fused(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, epilogue: int = EPI_NONE,
               norm_weight: Optional[torch.Tensor] = None, sumsq_in: Optional[torch.Tensor] = None, eps: float = 1e-5,
               residual: Optional[torch.Tensor] = None, want_sumsq: bool = False,
               workspace: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None):
    """``gemv`` with a decoder block's surroundings folded in.

    ``norm_weight`` + ``sumsq_in`` (fp32 [B, K/16]): the product is taken with ``RMSNorm(x)``;
    ``residual`` ([B, N]): ``y = dtype(dtype(x W^T + bias) + residual)`` (``out`` may be ``residual``);
    ``want_sumsq``: also returns fp32 [B, ceil(N/16)] sums of squares of ``y``, the next norm's ``sumsq_in``.
    Returns ``y`` or ``(y, sumsq)``."""
    dev = _require_gpu(x, w, bias, workspace, norm_weight, sumsq_in, residual, out)
    dt = _decode_dtype("gemv_fused", x, w, bias)
    B, N, K = _gemv_shapes("gemv_fused", x, w, bias)
    x, w = _contig(x), _contig(w)
    n_out = N // 2 if epilogue == EPI_SWIGLU else N
    if norm_weight is not None:
        if sumsq_in is None or sumsq_in.dtype != torch.float32 or tuple(sumsq_in.shape) != (B, K // 16) \
                or not sumsq_in.is_contiguous():
            raise ValueError(f"gemv_fused: sumsq_in must be contiguous fp32 [{B}, {K // 16}]")
        if norm_weight.dtype != dt or norm_weight.numel() != K or not norm_weight.is_contiguous():
            raise ValueError(f"gemv_fused: norm_weight must be contiguous {dt} [{K}]")
    if residual is not None and (residual.dtype != dt or tuple(residual.shape) != (B, n_out) or not residual.is_contiguous()):
        raise ValueError(f"gemv_fused: residual must be contiguous {dt} [{B}, {n_out}]")
    if out is None:
        out = torch.empty((B, n_out), dtype=dt, device=dev)
    elif out.dtype != dt or tuple(out.shape) != (B, n_out) or not out.is_contiguous():
        raise ValueError(f"gemv_fused: out must be contiguous {dt} [{B}, {n_out}]")
    sumsq = torch.empty((B, (N + 15) // 16), dtype=torch.float32, device=dev) if want_sumsq else None
    wbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_gemv_fused(_p(x), _p(w), _p(bias), _p(out), _p(norm_weight), _p(sumsq_in), float(eps),
                                             _p(residual), _p(sumsq), _p(workspace), wbytes, B, N, K, epilogue,
                                             _DTYPES[dt], _stream(dev)), "mtp_gemv_fused")
    return (out, sumsq) if want_sumsq else out


def argmax_workspace(B: int, N: int, K: int, dev: torch.device) -> torch.Tensor:
    """Scratch for ``gemv_argmax`` on shapes up to [B, K] x [N, K] (nothing in it needs clearing)."""
    need = _lib.lib().mtp_gemv_argmax_workspace_bytes(B, N, K)
    return torch.empty((max(int(need), 8),), dtype=torch.uint8, device=dev)


def gemv_argmax(x: torch.Tensor, w: torch.Tensor, workspace: Optional[torch.Tensor] = None):
    """-> (idx int64 [B], maxval fp32 [B]) without materialising the logits."""
    dev = _require_gpu(x, w, workspace)
    dt = _decode_dtype("gemv_argmax", x, w)
    B, N, K = _gemv_shapes("gemv_argmax", x, w, None)
    x, w = _contig(x), _contig(w)
    need = _lib.lib().mtp_gemv_argmax_workspace_bytes(B, N, K)
    if workspace is None:
        workspace = argmax_workspace(B, N, K, dev)
    idx = torch.empty((B,), dtype=torch.int64, device=dev)
    val = torch.empty((B,), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_gemv_argmax(_p(x), _p(w), _p(idx), _p(val), _p(workspace),
                                              workspace.numel() * workspace.element_size(), B, N, K,
                                              _DTYPES[dt], _stream(dev)), "mtp_gemv_argmax")
    return idx, val


def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    dev = _require_gpu(logits)
    l2 = _contig(logits).view(-1, logits.shape[-1])
    idx = torch.empty((l2.shape[0],), dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_argmax_rows(_p(l2), _p(idx), l2.shape[0], l2.shape[1], _dt(l2), _stream(dev)),
                   "mtp_argmax_rows")
    return idx.view(logits.shape[:-1])


def sample_top_k_top_p(logits: torch.Tensor, temperature: float = 1.0, top_k: int = 0, top_p: float = 0.0,
                       uniforms: Optional[torch.Tensor] = None, want_filtered: bool = False,
                       workspace: Optional[torch.Tensor] = None):
    """-> (tokens int64 [B] or None, filtered fp32 [B, V] or None).

    tokens are drawn when ``uniforms`` (fp32 [B], values in [0, 1)) is given."""
    dev = _require_gpu(logits, uniforms, workspace)
    if logits.dim() != 2:
        raise ValueError("sample_top_k_top_p takes [B, V] logits")
    logits = _contig(logits)
    B, V = logits.shape
    tokens = filtered = None
    if uniforms is not None:
        uniforms = _contig(uniforms.to(torch.float32)).view(-1)
        if uniforms.numel() != B:
            raise ValueError(f"uniforms has {uniforms.numel()} entries for {B} rows")
        tokens = torch.empty((B,), dtype=torch.int64, device=dev)
    if want_filtered:
        filtered = torch.empty((B, V), dtype=torch.float32, device=dev)
    if tokens is None and filtered is None:
        raise ValueError("nothing to compute: give uniforms and/or want_filtered=True")
    lib = _lib.lib()
    need = int(lib.mtp_sample_workspace_bytes(B))
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        workspace = torch.empty((max(need, 8),), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(lib.mtp_sample_top_k_top_p(_p(logits), _dt(logits), B, V, float(temperature), int(top_k),
                                              float(top_p), _p(uniforms), _p(tokens), _p(filtered), _p(workspace),
                                              workspace.numel() * workspace.element_size(), _stream(dev)),
                   "mtp_sample_top_k_top_p")
    return tokens, filtered


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None,
            want_residual: bool = False):
    """-> y, or (y, h) with ``want_residual``: h = x (+ residual), y = weight * (h * rsqrt(mean(h^2) + eps))."""
    dev = _require_gpu(x, weight, residual)
    x = _contig(x)
    dim = x.shape[-1]
    if weight.shape != (dim,) or weight.dtype != x.dtype:
        raise ValueError(f"rmsnorm: weight {tuple(weight.shape)} {weight.dtype} for rows of {dim} {x.dtype}")
    if residual is not None:
        residual = _contig(residual)
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise ValueError("rmsnorm: residual must match x")
    y = torch.empty_like(x)
    h = torch.empty_like(x) if want_residual else None
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_rmsnorm(_p(x), _p(residual), _p(_contig(weight)), _p(y), _p(h), x.numel() // dim, dim,
                                          float(eps), _dt(x), _stream(dev)), "mtp_rmsnorm")
    return (y, h) if want_residual else y


def rope_kv_append(qkv: torch.Tensor, cos_table: torch.Tensor, sin_table: torch.Tensor, positions: torch.Tensor,
                   k_cache: torch.Tensor, v_cache: torch.Tensor, n_q_heads: int) -> torch.Tensor:
    """Rotates the new q and k heads of ``qkv`` [B, (n_q + 2 n_kv) * 128], writes k and v into row
    ``positions[b]`` of the caches [B, n_kv, max_len, 128] and returns the rotated q [B, n_q, 128]."""
    dev = _require_gpu(qkv, cos_table, sin_table, positions, k_cache, v_cache)
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("rope_kv_append: caches must be contiguous [B, n_kv_heads, max_len, head_dim] of one shape")
    B, n_kv, max_len, hd = k_cache.shape
    qkv = _contig(qkv)
    if qkv.shape != (B, (n_q_heads + 2 * n_kv) * hd):
        raise ValueError(f"rope_kv_append: qkv {tuple(qkv.shape)} for {n_q_heads}+2*{n_kv} heads of {hd}")
    if cos_table.shape != sin_table.shape or cos_table.dim() != 2 or cos_table.shape[1] != hd:
        raise ValueError("rope_kv_append: cos / sin tables must be [max_positions, head_dim]")
    for t in (cos_table, sin_table, k_cache, v_cache):
        if t.dtype != qkv.dtype:
            raise ValueError("rope_kv_append: all tensors must share the dtype of qkv")
    if positions.dtype != torch.int64 or positions.numel() != B:
        raise ValueError("rope_kv_append: positions must be int64 [B]")
    q = torch.empty((B, n_q_heads, hd), dtype=qkv.dtype, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_rope_kv_append(_p(qkv), _p(_contig(cos_table)), _p(_contig(sin_table)),
                                                 _p(_contig(positions)), _p(q), _p(k_cache), _p(v_cache), B,
                                                 n_q_heads, n_kv, hd, max_len, cos_table.shape[0], _dt(qkv),
                                                 _stream(dev)), "mtp_rope_kv_append")
    return q


def attn_decode_workspace_bytes(B: int, n_q_heads: int, n_kv_heads: int, len_bound: int) -> int:
    return int(_lib.lib().mtp_attn_decode_workspace_bytes(B, n_q_heads, n_kv_heads, len_bound))


def attn_workspace(B: int, n_q_heads: int, n_kv_heads: int, len_bound: int, device) -> torch.Tensor:
    """Zero-filled scratch for ``attn_decode`` / ``attn_decode_append`` (the kernels need its head zero before
    the first use and leave it zero)."""
    return torch.zeros((max(attn_decode_workspace_bytes(B, n_q_heads, n_kv_heads, len_bound), 16),), dtype=torch.uint8,
                       device=device)


def _attn_workspace(workspace, B, n_q, n_kv, len_bound, dev):
    need = attn_decode_workspace_bytes(B, n_q, n_kv, len_bound)
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = attn_workspace(B, n_q, n_kv, len_bound, dev)
    return workspace


def attn_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, lens: torch.Tensor,
                scale: Optional[float] = None, len_bound: Optional[int] = None,
                workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of one new position per row over the first ``lens[b]`` cached tokens.
    q [B, n_q, 128], caches [B, n_kv, max_len, 128] -> [B, n_q, 128]."""
    dev = _require_gpu(q, k_cache, v_cache, lens, workspace)
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("attn_decode: caches must be contiguous [B, n_kv_heads, max_len, head_dim] of one shape")
    B, n_kv, max_len, hd = k_cache.shape
    q = _contig(q)
    if q.dim() != 3 or q.shape[0] != B or q.shape[2] != hd:
        raise ValueError(f"attn_decode: q {tuple(q.shape)} against caches {tuple(k_cache.shape)}")
    if not (q.dtype == k_cache.dtype == v_cache.dtype):
        raise ValueError("attn_decode: q and the caches must share a dtype")
    if lens.dtype != torch.int64 or lens.numel() != B:
        raise ValueError("attn_decode: lens must be int64 [B]")
    n_q = q.shape[1]
    len_bound = max_len if len_bound is None else int(len_bound)
    scale = hd ** -0.5 if scale is None else float(scale)
    lib = _lib.lib()
    workspace = _attn_workspace(workspace, B, n_q, n_kv, len_bound, dev)
    out = torch.empty_like(q)
    wbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    with torch.cuda.device(dev):
        _lib.check(lib.mtp_attn_decode(_p(q), _p(k_cache), _p(v_cache), _p(_contig(lens)), _p(out), _p(workspace),
                                       wbytes, B, n_q, n_kv, hd, max_len, len_bound, scale, _dt(q), _stream(dev)),
                   "mtp_attn_decode")
    return out


def attn_decode_append(qkv: torch.Tensor, cos_table: torch.Tensor, sin_table: torch.Tensor, positions: torch.Tensor,
                       k_cache: torch.Tensor, v_cache: torch.Tensor, n_q_heads: int, scale: Optional[float] = None,
                       len_bound: Optional[int] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``rope_kv_append`` then ``attn_decode`` over ``positions + 1`` tokens, as one launch.
    ``workspace``: from ``attn_workspace`` (zero-filled once, reusable)."""
    dev = _require_gpu(qkv, cos_table, sin_table, positions, k_cache, v_cache, workspace)
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("attn_decode_append: caches must be contiguous [B, n_kv_heads, max_len, head_dim] of one shape")
    B, n_kv, max_len, hd = k_cache.shape
    qkv = _contig(qkv)
    if qkv.shape != (B, (n_q_heads + 2 * n_kv) * hd):
        raise ValueError(f"attn_decode_append: qkv {tuple(qkv.shape)} for {n_q_heads}+2*{n_kv} heads of {hd}")
    if cos_table.shape != sin_table.shape or cos_table.dim() != 2 or cos_table.shape[1] != hd:
        raise ValueError("attn_decode_append: cos / sin tables must be [max_positions, head_dim]")
    for t in (cos_table, sin_table, k_cache, v_cache):
        if t.dtype != qkv.dtype:
            raise ValueError("attn_decode_append: all tensors must share the dtype of qkv")
    if positions.dtype != torch.int64 or positions.numel() != B:
        raise ValueError("attn_decode_append: positions must be int64 [B]")
    len_bound = max_len if len_bound is None else int(len_bound)
    scale = hd ** -0.5 if scale is None else float(scale)
    workspace = _attn_workspace(workspace, B, n_q_heads, n_kv, len_bound, dev)
    out = torch.empty((B, n_q_heads, hd), dtype=qkv.dtype, device=dev)
    wbytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mtp_attn_decode_append(_p(qkv), _p(_contig(cos_table)), _p(_contig(sin_table)),
                                                     _p(_contig(positions)), _p(k_cache), _p(v_cache), _p(out),
                                                     _p(workspace), wbytes, B, n_q_heads, n_kv, hd, max_len,
                                                     cos_table.shape[0], len_bound, scale, _dt(qkv), _stream(dev)),
                   "mtp_attn_decode_append")
    return out

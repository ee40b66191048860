"""Python faces of the HIP kernels.

Each function checks on the host that the operands have the shapes, types and
placement its kernel and grid assume, then launches on torch's current stream.
Tensors are torch tensors on a HIP device; torch is used for memory and
streams only.  Nothing here falls back to the CPU or to a library routine:
a missing library or a refused size raises
:class:`~sonicboom_amd.ops.library.KernelLibraryError`.
"""
from __future__ import annotations

import contextlib
import math
import threading

from typing import Optional

import torch

from . import library
from .library import KernelLibraryError, check

class _Hints(threading.local):
    """Choices a test or a measurement imposes on the launchers, for the calls of its own thread
    inside a ``with`` block; every kernel call passes them as arguments (the library keeps no
    such state)."""
    few_rows_kernel = None      # "stream", "skinny", "tiled" or None
    stream = 0                  # waves | slices << 8 of the weight-streaming product
    tile_shape = -1             # of the tiled product
    decode_pages = 0            # pages per wave of decode attention


_hints = _Hints()

from ..csrc.header import PAGE          # tokens per cache page: SB_PAGE of csrc/sb_hip.h
MAX_CANDIDATES = 256

_DT = {torch.float32: 0, torch.bfloat16: 1}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelLibraryError(f"kernels take float32 and bfloat16 tensors, not {t.dtype}") from None


def _dev(*ts) -> None:
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelLibraryError("kernel operands must live on the GPU (there is no CPU path)")
        if not t.is_contiguous():
            raise KernelLibraryError("kernel operands must be contiguous")


def _on_gpu(*ts) -> None:
    """For operands that may be views of wider rows: on the GPU, layout checked by the caller."""
    for t in ts:
        if t is not None and not t.is_cuda:
            raise KernelLibraryError("kernel operands must live on the GPU (there is no CPU path)")


def _i32(t: torch.Tensor, n: int, what: str) -> None:
    if t.dtype != torch.int32 or t.numel() < n:
        raise KernelLibraryError(f"{what} must be int32 with at least {n} elements")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle.  (torch's own accessor for the raw handle where it has one:
    building a Stream object for every launch cost 8 us of a launch's 14 on the host.)"""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


# --------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rows of ``table`` [vocab, width] named by int32 ``ids`` [n], as float32."""
    _dev(table, ids, out)
    if table.dim() != 2:
        raise KernelLibraryError("embedding table must be [vocab, width]")
    n = ids.numel()
    _i32(ids, n, "token ids")
    vocab, width = table.shape
    if out is None:
        out = torch.empty((n, width), dtype=torch.float32, device=table.device)
    elif out.dtype != torch.float32 or out.numel() != n * width:
        raise KernelLibraryError("embedding output must be float32 [n, width]")
    lib = library.core()
    check(lib.sb_embed(_p(out), _p(table), _dt(table), _p(ids), n, width, vocab, _stream()))
    return out


def rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype,
            rows: Optional[torch.Tensor] = None, groups: int = 1) -> torch.Tensor:
    """RMS norm of float32 rows ``x`` [n, width]; ``rows`` (int32) picks and orders source rows;
    ``groups`` > 1: each of that many equal consecutive parts of a row by its own root mean square."""
    _dev(x, weight, rows)
    if x.dtype != torch.float32 or x.dim() != 2:
        raise KernelLibraryError("rmsnorm input must be float32 [rows, width]")
    width = x.shape[1]
    if weight is not None and weight.numel() != width:
        raise KernelLibraryError(f"rmsnorm weight has {weight.numel()} elements, the rows have {width}")
    n = x.shape[0] if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, n, "row index")
    y = torch.empty((n, width), dtype=out_dtype, device=x.device)
    lib = library.core()
    if groups != 1:
        if groups < 1 or width % groups:
            raise KernelLibraryError(f"{groups} groups do not divide a row of {width}")
        check(lib.sb_rmsnorm_grouped(_p(y), _dt(y), _p(x), _p(weight), _dt(weight) if weight is not None else 0,
                                     _p(rows), n, width, int(groups), float(eps), _stream()))
        return y
    check(lib.sb_rmsnorm(_p(y), _dt(y), _p(x), _p(weight), _dt(weight) if weight is not None else 0,
                         _p(rows), n, width, float(eps), _stream()))
    return y


def gemm_plain(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], resid: Optional[torch.Tensor],
               out_dtype: torch.dtype, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x w^T (+bias) (+resid) by the plain tiled kernel; any sizes, f32 or bf16 operands."""
    _dev(x, w, bias, resid, out)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelLibraryError(f"gemm shapes do not match: x {tuple(x.shape)}, w {tuple(w.shape)}")
    t, k = x.shape
    n = w.shape[0]
    if bias is not None and bias.numel() != n:
        raise KernelLibraryError(f"bias has {bias.numel()} elements, the product has {n} columns")
    if resid is not None and (resid.dtype != torch.float32 or tuple(resid.shape) != (t, n)):
        raise KernelLibraryError("the residual must be float32 and shaped like the product")
    if out is None:
        out = torch.empty((t, n), dtype=out_dtype, device=x.device)
    elif out.dtype != out_dtype or tuple(out.shape) != (t, n):
        raise KernelLibraryError("gemm output buffer has the wrong shape or type")
    lib = library.core()
    check(lib.sb_gemm(_p(out), _dt(out), _p(x), _dt(x), _p(w), _dt(w), _p(bias),
                      _dt(bias) if bias is not None else 0, _p(resid), t, n, k, _stream()))
    return out


GATES = {"silu": 1, "gelu_tanh": 2, "relu": 3}      # sb_gate of csrc/sb_hip.h


def gate_code(activation) -> int:
    """The kernels' number of a gate activation given by name (or already by number)."""
    if isinstance(activation, bool):
        return 1 if activation else 0
    if isinstance(activation, int):
        return activation
    try:
        return GATES[activation]
    except KeyError:
        raise KernelLibraryError(f"unknown gate activation {activation!r}; known: {sorted(GATES)}") from None


def gate_mul(gu: torch.Tensor, out_dtype: torch.dtype, activation="silu") -> torch.Tensor:
    """act(gu[:, :w]) * gu[:, w:] for gu [n, 2w]; ``activation``: "silu" or "gelu_tanh"."""
    _dev(gu)
    if gu.dim() != 2 or gu.shape[1] % 2:
        raise KernelLibraryError("gate_mul input must be [rows, 2*width]")
    n, w2 = gu.shape
    out = torch.empty((n, w2 // 2), dtype=out_dtype, device=gu.device)
    lib = library.core()
    check(lib.sb_gate_mul(_p(out), _dt(out), _p(gu), _dt(gu), n, w2 // 2, gate_code(activation), _stream()))
    return out


def silu_mul(gu: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """silu(gu[:, :w]) * gu[:, w:] for gu [n, 2w]."""
    return gate_mul(gu, out_dtype, "silu")


def add_into(resid: torch.Tensor, y: torch.Tensor) -> None:
    """resid += y (resid float32)."""
    _dev(resid, y)
    if resid.dtype != torch.float32 or resid.numel() != y.numel():
        raise KernelLibraryError("add_into needs a float32 residual and an addend of the same size")
    lib = library.core()
    check(lib.sb_add_into(_p(resid), _p(y), _dt(y), resid.numel(), _stream()))


def add_scaled(resid: torch.Tensor, y: torch.Tensor, scale: float) -> None:
    """resid += scale * y (float32 residual stream, in place)."""
    _dev(resid, y)
    if resid.dtype != torch.float32 or resid.numel() != y.numel():
        raise KernelLibraryError("add_scaled needs a float32 residual and an addend of the same size")
    check(library.core().sb_add_scaled(_p(resid), _p(y), _dt(y), float(scale), resid.numel(), _stream()))


ACTIVATIONS = {"silu": 1, "gelu_tanh": 2, "xielu": 3, "gelu_erf": 4, "relu_sq": 5}      # sb_act of csrc/sb_hip.h


def activate(x: torch.Tensor, out_dtype: torch.dtype, activation: str, params: Optional[torch.Tensor] = None) -> torch.Tensor:
    """act(x) element by element; ``params``: the numbers an activation reads from memory (xIELU's
    two, of which the kernel takes the softplus itself)."""
    _dev(x, params)
    try:
        kind = ACTIVATIONS[activation]
    except KeyError:
        raise KernelLibraryError(f"unknown activation {activation!r}; known: {sorted(ACTIVATIONS)}") from None
    if activation == "xielu" and (params is None or params.numel() != 2):
        raise KernelLibraryError("xIELU takes two numbers")
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    check(library.core().sb_activate(_p(out), _dt(out), _p(x), _dt(x), x.numel(), kind, _p(params),
                                     _dt(params) if params is not None else 0, _stream()))
    return out


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    _dev(x)
    if x.dtype == dtype:
        return x
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    lib = library.core()
    check(lib.sb_cast(_p(out), _dt(out), _p(x), _dt(x), x.numel(), _stream()))
    return out


def rmsnorm_pair(x: torch.Tensor, weight1: Optional[torch.Tensor], weight2: Optional[torch.Tensor], eps: float,
                 out_dtype: torch.dtype, second: bool = True):
    """Two RMS norms of the same float32 rows in one pass: (x inv) w1 and (x inv) w2 with one root mean
    square for both.  ``x`` may be a view of wider rows (columns of a product's result): its last axis
    dense, its rows any distance apart.  ``second`` false: the first alone (returns (y1, None))."""
    _dev(weight1, weight2)
    _on_gpu(x)
    if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
        raise KernelLibraryError("the norm's input must be float32 [rows, width], dense along a row")
    n, width = x.shape
    for w in (weight1, weight2):
        if w is not None and w.numel() != width:
            raise KernelLibraryError(f"a norm weight has {w.numel()} elements, the rows have {width}")
    if weight1 is not None and weight2 is not None and weight1.dtype != weight2.dtype:
        raise KernelLibraryError("the two norm weights must be of one type")
    wt = weight1 if weight1 is not None else weight2
    y1 = torch.empty((n, width), dtype=out_dtype, device=x.device)
    y2 = torch.empty((n, width), dtype=out_dtype, device=x.device) if second else None
    check(library.core().sb_rmsnorm_pair(_p(y1), _p(y2), _DT[out_dtype], _p(x), x.stride(0) if n > 1 else width, _p(weight1),
                                         _p(weight2), _dt(wt) if wt is not None else 0, n, width, float(eps), _stream()))
    return y1, y2


def sigmoid_mul_(x: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """x *= sigmoid(gate) in place, element by element: ``x`` [rows, width] dense, ``gate`` float32
    [rows, width], possibly a view of wider rows."""
    _dev(x)
    _on_gpu(gate)
    if x.dim() != 2 or not x.is_contiguous() or gate.dtype != torch.float32 or gate.shape != x.shape or gate.stride(1) != 1:
        raise KernelLibraryError("sigmoid_mul_ takes dense rows and a float32 gate of the same shape")
    n, width = x.shape
    check(library.core().sb_sigmoid_mul(_p(x), _dt(x), _p(gate), gate.stride(0) if n > 1 else width, n, width, _stream()))
    return x


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap tanh(x / cap) in place (float32)."""
    _dev(x)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelLibraryError("softcap_ takes dense float32 values")
    check(library.core().sb_softcap(_p(x), float(cap), x.numel(), _stream()))
    return x


def _check_cache(k_cache, v_cache, heads_kv, head_dim):
    if k_cache.dim() != 4 or v_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (heads_kv, PAGE, head_dim) \
            or tuple(v_cache.shape[1:]) != (heads_kv, head_dim, PAGE) or k_cache.shape[0] != v_cache.shape[0] \
            or k_cache.dtype != v_cache.dtype:
        raise KernelLibraryError(
            f"cache must be keys [pages, {heads_kv}, {PAGE}, {head_dim}] and values "
            f"[pages, {heads_kv}, {head_dim}, {PAGE}], found {tuple(k_cache.shape)} and {tuple(v_cache.shape)}")


def _check_rows(row_pos, row_seq, page_table, n_rows):
    _i32(row_pos, n_rows, "row positions")
    _i32(row_seq, n_rows, "row sequence index")
    if page_table.dtype != torch.int32 or page_table.dim() != 2:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")


def rope_kv_store(qkv: torch.Tensor, q_dtype: torch.dtype, inv_freq: Optional[torch.Tensor],
                  freq_factors: Optional[torch.Tensor], rot_dims: int, row_pos: torch.Tensor,
                  row_seq: torch.Tensor, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  page_table: Optional[torch.Tensor], heads_q: int, heads_kv: int, head_dim: int,
                  bias: Optional[torch.Tensor] = None, v_dim: int = 0, magnitude: float = 1.0) -> torch.Tensor:
    """Rotate queries and keys of ``qkv`` [n, (hq+2hkv)*hd], return the queries
    [n, hq*hd] in ``q_dtype`` and store keys and values in the paged cache.
    ``heads_kv`` = 0 (and no cache) for a layer that stores nothing.  ``qkv`` may be
    [slices, n, width]: partial sums of the projection, added here in ascending order;
    ``bias`` (float32 [width]) is added after them.  ``v_dim``: the size of a value head when it
    is not the keys' (the row is then [hq*hd | hkv*hd | hkv*v_dim]); ``magnitude`` multiplies every
    cosine and sine."""
    _dev(qkv, inv_freq, freq_factors, row_pos, row_seq, k_cache, v_cache, page_table, bias)
    n_slices = 1
    if qkv.dim() == 3:
        n_slices = qkv.shape[0]
        qkv = qkv.view(-1, qkv.shape[2])
    n = qkv.shape[0] // n_slices
    v_dim = int(v_dim) or head_dim
    need = (heads_q + heads_kv) * head_dim + heads_kv * v_dim
    if qkv.dim() != 2 or qkv.shape[1] < need:
        raise KernelLibraryError(f"qkv rows have {qkv.shape[1]} elements, {need} are needed")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() < need):
        raise KernelLibraryError("the qkv bias must be float32 and cover a whole row")
    if inv_freq is not None:
        if inv_freq.dtype != torch.float32 or inv_freq.numel() != rot_dims // 2:
            raise KernelLibraryError("inv_freq must be float32 [rot_dims/2]")
        if freq_factors is not None and (freq_factors.dtype != torch.float32 or freq_factors.numel() < rot_dims // 2):
            raise KernelLibraryError("freq_factors must be float32 [rot_dims/2]")
    _i32(row_pos, n, "row positions")
    max_pages = n_pages = 0
    if heads_kv > 0:
        _check_cache_kv(k_cache, v_cache, heads_kv, head_dim, v_dim)
        _check_rows(row_pos, row_seq, page_table, n)
        max_pages, n_pages = page_table.shape[1], k_cache.shape[0]
    q = torch.empty((n, heads_q * head_dim), dtype=q_dtype, device=qkv.device)
    lib = library.core()
    check(lib.sb_rope_kv_store_sized(
        _p(q), _dt(q), _p(qkv), _dt(qkv), qkv.shape[1], n_slices, _p(bias), _p(inv_freq), _p(freq_factors), rot_dims,
        _p(row_pos), _p(row_seq), _p(k_cache), _p(v_cache), _dt(k_cache) if k_cache is not None else 0,
        _p(page_table), max_pages, n_pages, n, heads_q, heads_kv, head_dim, v_dim, float(magnitude), _stream()))
    return q


def attention_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                    row_pos: torch.Tensor, row_seq: torch.Tensor, heads_q: int, heads_kv: int, head_dim: int,
                    scale: float, window: int) -> torch.Tensor:
    """Attention of rows ``q`` [n, hq*hd] over the cache, by the plain kernel."""
    _dev(q, k_cache, v_cache, page_table, row_pos, row_seq)
    n = q.shape[0]
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim:
        raise KernelLibraryError(f"queries must be [rows, {heads_q * head_dim}]")
    _check_cache(k_cache, v_cache, heads_kv, head_dim)
    _check_rows(row_pos, row_seq, page_table, n)
    out = torch.empty((n, heads_q * head_dim), dtype=q.dtype, device=q.device)
    lib = library.core()
    check(lib.sb_attention(_p(out), _p(q), _dt(q), q.shape[1], _p(k_cache), _p(v_cache), _dt(k_cache),
                           _p(page_table), page_table.shape[1], k_cache.shape[0], _p(row_pos), _p(row_seq),
                           n, heads_q, heads_kv, head_dim, float(scale), int(window), _stream()))
    return out


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """First maximum of every row of float32 ``logits`` [n, vocab], int32 [n]."""
    _dev(logits, out)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelLibraryError("logits must be float32 [rows, vocab]")
    n, vocab = logits.shape
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    else:
        _i32(out, n, "argmax output")
    lib = library.core()
    parts = lib.sb_argmax_parts(vocab)
    pv = pi = None
    if parts > 1:
        pv = torch.empty((n * parts,), dtype=torch.float32, device=logits.device)
        pi = torch.empty((n * parts,), dtype=torch.int32, device=logits.device)
    check(lib.sb_argmax(_p(out), _p(logits), n, vocab, _p(pv), _p(pi), _stream()))
    return out


def penalize(logits: torch.Tensor, item_row: torch.Tensor, item_token: torch.Tensor, item_count: torch.Tensor,
             repeat_penalty: float, presence_penalty: float, frequency_penalty: float, exact: bool) -> None:
    """Apply sampling penalties in place for (row, token, count) triples."""
    _dev(logits, item_row, item_token, item_count)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelLibraryError("logits must be float32 [rows, vocab]")
    n = item_row.numel()
    for t, what in ((item_row, "item rows"), (item_token, "item tokens"), (item_count, "item counts")):
        _i32(t, n, what)
    lib = library.core()
    check(lib.sb_penalize(_p(logits), logits.shape[1], _p(item_row), _p(item_token), _p(item_count), n,
                          float(repeat_penalty), float(presence_penalty), float(frequency_penalty),
                          1 if exact else 0, _stream()))


def top_candidates(logits: torch.Tensor, temperature: float, k: int = MAX_CANDIDATES):
    """The ``k`` best candidates of every row by z = logit / temperature:
    (ids int32 [n,k], z float32 [n,k]) ordered by (z descending, id ascending)."""
    _dev(logits)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelLibraryError("logits must be float32 [rows, vocab]")
    n, vocab = logits.shape
    ids = torch.empty((n, k), dtype=torch.int32, device=logits.device)
    z = torch.empty((n, k), dtype=torch.float32, device=logits.device)
    lib = library.core()
    words = lib.sb_top_candidates_scratch(n, vocab)
    scratch = torch.empty((words,), dtype=torch.int64, device=logits.device) if words else None
    check(lib.sb_top_candidates(_p(ids), _p(z), _p(logits), n, vocab, k, float(temperature), _p(scratch), _stream()))
    return ids, z


def mask_logits(logits: torch.Tensor, bitmaps: torch.Tensor) -> None:
    """The mask of constrained decoding, in place: float32 ``logits`` [rows, vocab] become -inf
    wherever the row's bitmap (uint8 [rows, bytes]: bit i & 7 of byte i >> 3 for id i; ids past the
    bitmap are not allowed) does not allow the id."""
    _dev(logits, bitmaps)
    if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
        raise KernelLibraryError("logits must be contiguous float32 [rows, vocab]")
    if bitmaps.dtype != torch.uint8 or bitmaps.dim() != 2 or bitmaps.shape[0] != logits.shape[0] \
            or bitmaps.shape[1] == 0 or not bitmaps.is_contiguous():
        raise KernelLibraryError("bitmaps must be contiguous uint8 [rows, bytes], a row for every row of logits")
    check(library.core().sb_mask_logits(_p(logits), logits.shape[0], logits.shape[1], _p(bitmaps),
                                        bitmaps.shape[1], _stream()))


def draw(cand_ids: torch.Tensor, cand_z: torch.Tensor, positions, top_k: int, log_min_p: Optional[float],
         top_p: Optional[float], seed: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row (int32 [n]; -1 where no candidate is kept) from the candidates that
    :func:`top_candidates` wrote: the window of 30 below the best z, top-k (0: off), min-p
    (``log_min_p`` = ln(min_p) rounded to float32, None: off), top-p (a float64, None: off) and
    the Gumbel-max draw under (seed, position of the row's new token, candidate id).
    ``positions``: one absolute position per row, a sequence or an int64 tensor on the device; or
    an int32 tensor on the device of each row's cached length before the step, whose new token then
    takes position length + 1 (a decode step's own bookkeeping: nothing comes from the host)."""
    _dev(cand_ids, cand_z)
    if cand_ids.dtype != torch.int32 or cand_z.dtype != torch.float32 or cand_ids.dim() != 2 \
            or tuple(cand_ids.shape) != tuple(cand_z.shape):
        raise KernelLibraryError("candidates must be int32 ids and float32 z of one shape [rows, k]")
    n, k = cand_ids.shape
    if not torch.is_tensor(positions):
        positions = torch.tensor([int(q) for q in positions], dtype=torch.int64).to(cand_ids.device)
    _dev(positions, out)
    if positions.dtype not in (torch.int64, torch.int32) or positions.numel() != n or not positions.is_contiguous():
        raise KernelLibraryError("positions must be int64 (or int32 lengths), contiguous, one per row")
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=cand_ids.device)
    elif out.dtype != torch.int32 or out.numel() != n or not out.is_contiguous():
        raise KernelLibraryError("the tokens' buffer must be contiguous int32, one per row")
    lib = library.core()
    entry = lib.sb_draw if positions.dtype == torch.int64 else lib.sb_draw_after
    check(entry(_p(out), _p(cand_ids.contiguous()), _p(cand_z.contiguous()), _p(positions),
                n, k, int(top_k), 0 if log_min_p is None else 1,
                0.0 if log_min_p is None else float(log_min_p), 0 if top_p is None else 1,
                0.0 if top_p is None else float(top_p), int(seed) & 0xFFFFFFFFFFFFFFFF, _stream()))
    return out


def read_bandwidth(n_bytes: int = 1 << 30, blocks: int = 512, repeats: int = 5, device="cuda:0") -> float:
    """Bytes a second that a plain streaming read of ``n_bytes`` reaches on this GPU (the best of
    ``repeats`` passes over a buffer that the caches do not hold): what "achievable" means beside
    the published peak in a bandwidth report."""
    n_bytes = max(16, n_bytes // 16 * 16)
    src = torch.zeros((n_bytes // 4,), dtype=torch.int32, device=device)
    sink = torch.zeros((4,), dtype=torch.int32, device=device)
    lib = library.core()
    best = 0.0
    for _ in range(repeats + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        check(lib.sb_read_probe(_p(sink), _p(src), n_bytes, int(blocks), _stream()))
        e1.record()
        e1.synchronize()
        best = max(best, n_bytes / (e0.elapsed_time(e1) * 1e-3))
    return best


_RANDOM_KINDS = {torch.float32: 0, torch.bfloat16: 1, torch.float64: 2}


def random_normal(shape, seed: int, tensor_index: int, mean: float = 0.0, std: float = 1.0,
                  dtype: torch.dtype = torch.float32, device="cuda:0", first: int = 0) -> torch.Tensor:
    """Seeded normal values of ``shape`` drawn on the device: float32(mean + std z) as float32 or
    rounded to bfloat16, or (``dtype`` float64) the standard normals z themselves.  Element e of
    the tensor (counted from ``first``, a multiple of four) is a function of (seed, tensor_index,
    e) alone, the one the host computes in :mod:`sonicboom_amd.weights.random_stream`."""
    try:
        kind = _RANDOM_KINDS[dtype]
    except KeyError:
        raise KernelLibraryError(f"random values come as float32, bfloat16 or float64, not {dtype}") from None
    out = torch.empty(tuple(shape), dtype=dtype, device=device)
    if not out.is_cuda:
        raise KernelLibraryError("random values are drawn on the GPU (the host has its own function for them)")
    lib = library.core()
    with torch.cuda.device(out.device):
        check(lib.sb_random_normal(_p(out), kind, out.numel(), int(first), int(seed) & (2 ** 64 - 1),
                                   int(tensor_index), float(mean), float(std), _stream()))
    return out


# --------------------------------------------------------------------------
# dispatch between the plain kernels and the MFMA kernels
# --------------------------------------------------------------------------
SKINNY_MAX_ROWS = 64


def gemm_bf16_partial(x: torch.Tensor, w: torch.Tensor, packed_shape=None) -> Optional[torch.Tensor]:
    """The raw product x w^T of bfloat16 rows in K slices, float32 [slices, rows, out], for a
    consumer that adds the slices itself (:func:`reduce_resid_norm`, :func:`rope_kv_store`).
    Packed weights, up to 64 rows: the kernel whose waves split the output features and share
    the rows through LDS, with K cut over the grid so that the blocks fill the GPU.
    Packed weights, more rows: the tiled kernel with K cut over the grid, as long as the cut gives
    more than one slice (a narrow matrix and up to a few hundred rows, where one slice would leave
    most of the GPU without a tile; or a thousand or two, where tiles of 256 x 256 with K cut in
    two to four beat the whole product in smaller tiles).  Row-major weights, up to 64 rows: the kernel whose waves split K.  None when
    none applies: the caller then takes the whole product."""
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or x.dim() != 2:
        return None
    n, k = packed_shape if packed_shape is not None else (w.shape[0], w.shape[-1])
    t = x.shape[0]
    if x.shape[1] != k:
        raise KernelLibraryError(f"gemm shapes do not match: x {tuple(x.shape)}, w {(n, k)}")
    if t == 0 or k % 8 or x.data_ptr() % 16 or w.data_ptr() % 16:
        return None
    lib = library.core()
    which = _hints.few_rows_kernel
    if packed_shape is not None and t <= SKINNY_MAX_ROWS and which in (None, "stream"):
        slices = lib.sb_gemm_stream_slices(t, n, k, _hints.stream)
        partial = torch.empty((slices, t, n), dtype=torch.float32, device=x.device)
        check(lib.sb_gemm_stream_partial_bf16(_p(partial), _p(x), _p(w), t, n, k, _hints.stream, _stream()))
        return partial
    if packed_shape is not None and (t > SKINNY_MAX_ROWS or which == "tiled"):
        slices = lib.sb_gemm_mfma_slices(t, n, k, 1)
        if slices > 1 or t <= SKINNY_MAX_ROWS:
            partial = torch.empty((slices, t, n), dtype=torch.float32, device=x.device)
            check(lib.sb_gemm_mfma_partial_bf16(_p(partial), _p(x), _p(w), t, n, k, 1, _stream()))
            return partial
        return None
    if t > SKINNY_MAX_ROWS:
        return None
    slices = lib.sb_gemm_skinny_slices(t, n, k)
    partial = torch.empty((slices, t, n), dtype=torch.float32, device=x.device)
    check(lib.sb_gemm_skinny_partial_bf16(_p(partial), _p(x), _p(w), t, n, k, 1 if packed_shape is not None else 0,
                                          _stream()))
    return partial


def reduce_resid_norm(partial: torch.Tensor, bias: Optional[torch.Tensor], x: torch.Tensor,
                      norm_weight: Optional[torch.Tensor], eps: float, out_dtype: Optional[torch.dtype],
                      scale: float = 1.0, groups: int = 1) -> Optional[torch.Tensor]:
    """x += scale * (sum of the slices of ``partial`` [slices, rows, width] (+ bias)); when
    ``out_dtype`` is given also returns rmsnorm(x) * norm_weight in that type, the norm taken in
    ``groups`` parts of the row.  One pass over the row."""
    _dev(partial, bias, x, norm_weight)
    if partial.dim() != 3 or partial.dtype != torch.float32 or x.dtype != torch.float32 \
            or tuple(x.shape) != tuple(partial.shape[1:]):
        raise KernelLibraryError("reduce_resid_norm needs float32 slices [s, rows, width] and a residual [rows, width]")
    s_, t, width = partial.shape
    if bias is not None and bias.numel() != width:
        raise KernelLibraryError("bias does not match the row width")
    if norm_weight is not None and norm_weight.numel() != width:
        raise KernelLibraryError("norm weight does not match the row width")
    lib = library.core()
    y = torch.empty((t, width), dtype=out_dtype, device=x.device) if out_dtype is not None else None
    if scale != 1.0 or groups != 1:
        if groups < 1 or width % groups:
            raise KernelLibraryError(f"{groups} groups do not divide a row of {width}")
        check(lib.sb_reduce_scaled_group_norm(
            _p(y), _dt(y) if y is not None else 0, _p(x), _p(partial), s_, _p(bias),
            _dt(bias) if bias is not None else 0, float(scale), _p(norm_weight),
            _dt(norm_weight) if norm_weight is not None else 0, t, width, int(groups), float(eps),
            1 if out_dtype is not None else 0, _stream()))
        return y
    if width % 4 or width > lib.sb_reduce_resid_norm_max_width():
        raise KernelLibraryError(f"reduce_resid_norm takes widths in steps of 4 up to "
                                 f"{lib.sb_reduce_resid_norm_max_width()}, not {width}")
    check(lib.sb_reduce_resid_norm(_p(y), _dt(y) if y is not None else 0, _p(x), _p(partial), s_, _p(bias),
                                   _dt(bias) if bias is not None else 0, _p(norm_weight),
                                   _dt(norm_weight) if norm_weight is not None else 0, t, width, float(eps),
                                   1 if out_dtype is not None else 0, _stream()))
    return y


def reduce_resid_norm_ok(width: int, scale: float = 1.0, groups: int = 1) -> bool:
    if scale != 1.0 or groups != 1:
        return groups >= 1 and width % groups == 0       # the kernel for scaled sums and grouped norms: any width
    return width % 4 == 0 and width <= library.core().sb_reduce_resid_norm_max_width()


def pack_weight(w: torch.Tensor, gated: bool = False) -> torch.Tensor:
    """A bf16 projection weight [out, in] in the matrix-core tile layout: rows padded to 16, k to
    32, and every 16 x 32 tile stored as one 1 KB block in fragment order — lane l = 16 g + r of a
    wave owns elements [row r][k = 8 g .. 8 g + 7] at offset 8 l — tiles of one row block being
    consecutive in k.  A wave then reads a whole fragment with one contiguous 1 KB load and walks
    K through consecutive memory.  With ``gated`` the two halves [gate; up] are packed one after
    the other.  Returns a flat bf16 tensor."""
    if w.dim() != 2 or w.dtype != torch.bfloat16:
        raise KernelLibraryError("pack_weight takes a bfloat16 matrix [out, in]")
    halves = w.chunk(2, dim=0) if gated else (w,)
    out = []
    for h in halves:
        n, k = h.shape
        n16, k32 = (n + 15) // 16 * 16, (k + 31) // 32 * 32
        if (n16, k32) != (n, k):
            h = torch.nn.functional.pad(h, (0, k32 - k, 0, n16 - n))
        out.append(h.reshape(n16 // 16, 16, k32 // 32, 4, 8).permute(0, 2, 3, 1, 4).reshape(-1))
    return torch.cat(out).contiguous() if len(out) > 1 else out[0].contiguous()


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], resid: Optional[torch.Tensor],
              out_dtype: torch.dtype, out: Optional[torch.Tensor] = None, gated: bool = False,
              packed_shape=None) -> Optional[torch.Tensor]:
    """bfloat16 product on the matrix cores: y = x w^T (+bias) (+resid), or with ``gated``
    (True or "silu", or "gelu_tanh") y = act(x wg^T) * (x wu^T) for w = [wg; wu].  Up to 64 rows go to one of the two
    weight-streaming kernels, more to the tiled one.  ``packed_shape`` = (rows of w, inner size) says that ``w`` is
    in the layout of :func:`pack_weight`.  Returns None when the sizes fit neither kernel (an
    inner size that is not a multiple of 8): the caller then takes the plain kernel."""
    _dev(x, w, bias, resid, out)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return None
    w_rows, w_k = packed_shape if packed_shape is not None else (w.shape[0], w.shape[-1])
    if x.dim() != 2 or x.shape[1] != w_k or (packed_shape is None and w.dim() != 2):
        raise KernelLibraryError(f"gemm shapes do not match: x {tuple(x.shape)}, w {(w_rows, w_k)}")
    t, k = x.shape
    gate = gate_code(gated)
    n = w_rows // 2 if gated else w_rows
    if k % 8 or x.data_ptr() % 16 or w.data_ptr() % 16 or (gated and w_rows % 2):
        return None
    if bias is not None and bias.numel() != n:
        raise KernelLibraryError(f"bias has {bias.numel()} elements, the product has {n} columns")
    if resid is not None and (resid.dtype != torch.float32 or tuple(resid.shape) != (t, n)):
        raise KernelLibraryError("the residual must be float32 and shaped like the product")
    if out is None:
        out = torch.empty((t, n), dtype=out_dtype, device=x.device)
    elif out.dtype != out_dtype or tuple(out.shape) != (t, n):
        raise KernelLibraryError("gemm output buffer has the wrong shape or type")
    lib = library.core()
    bdt = _dt(bias) if bias is not None else 0
    packed = 1 if packed_shape is not None else 0
    # A wide packed matrix (enough 16-row tiles, or gate/up pairs of them, for STREAM_MIN_BLOCKS
    # blocks of four waves) and up to 128 rows: the kernel whose waves split the output features
    # and share the rows through LDS.  Other products of up to 64 rows: the kernel whose waves
    # split K and which can cut K over the grid as well.  The rest: the tiled kernel.
    which = _hints.few_rows_kernel
    if which is None:
        wave_units = -(-n // 16) if gated else -(-n // 32)
        which = "stream" if packed and wave_units >= 4 * STREAM_MIN_BLOCKS else "skinny"
        if t > SKINNY_MAX_ROWS and which == "stream":
            # 65 to 128 rows: the tiled kernel's 128 x 128 tiles do as well or better unless the
            # matrix is wide and their count leaves the last round over the 256 CUs nearly empty
            # (8,960 x 1,536 and 11,008 x 2,048 at 96 rows: 21 and 26 us tiled, 25 and 34 streamed)
            rounds = -(-n // (64 if gated else 128)) / 256.0
            if wave_units < 4 * STREAM_MIN_BLOCKS_MORE_ROWS or math.ceil(rounds) / rounds < 1.4:
                which = "tiled"
    if t <= STREAM_MAX_ROWS and which == "stream" and packed:
        check(lib.sb_gemm_stream_bf16(_p(out), _dt(out), _p(x), _p(w), _p(bias), bdt, _p(resid), t, n, k,
                                      gate, _hints.stream, _stream()))
    elif t <= SKINNY_MAX_ROWS and which != "tiled":
        need = lib.sb_gemm_skinny_scratch(t, n, k, gate)
        scratch = torch.empty((need,), dtype=torch.float32, device=x.device) if need else None
        check(lib.sb_gemm_skinny_bf16(_p(out), _dt(out), _p(x), _p(w), _p(bias), bdt, _p(resid), t, n, k,
                                      gate, packed, _p(scratch), need, _stream()))
    else:
        check(lib.sb_gemm_mfma_bf16(_p(out), _dt(out), _p(x), _p(w), _p(bias), bdt, _p(resid), t, n, k,
                                    gate, packed, _hints.tile_shape, _stream()))
    return out


def gemm_bf16_add_scaled(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], resid: torch.Tensor,
                         scale: float, packed_shape) -> bool:
    """resid += scale * (x w^T (+ bias)) in the tiled product's own epilogue (packed bfloat16 weights,
    more rows than the weight-streaming kernels take); False when the sizes are not the tiled kernel's,
    and the caller adds in a pass of its own."""
    _dev(x, w, bias, resid)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or packed_shape is None or x.dim() != 2:
        return False
    n, k = packed_shape
    t = x.shape[0]
    if t <= STREAM_MAX_ROWS or x.shape[1] != k or k % 8 or x.data_ptr() % 16 or w.data_ptr() % 16:
        return False
    if resid.dtype != torch.float32 or tuple(resid.shape) != (t, n) or (bias is not None and bias.numel() != n):
        raise KernelLibraryError("the residual must be float32 and shaped like the product")
    check(library.core().sb_gemm_mfma_scaled_bf16(_p(resid), 0, _p(x), _p(w), _p(bias), _dt(bias) if bias is not None else 0,
                                                  _p(resid), float(scale), t, n, k, 0, 1, _hints.tile_shape, _stream()))
    return True


@contextlib.contextmanager
def gemm_tile_shape(shape: Optional[int], path: Optional[str] = None):
    """For tests and measurements: inside the block the tiled products of this thread use tile
    shape ``shape`` (0: 128 x 128, 1: 256 x 128, 2: 256 x 256, 3: 128 x 256, 4: 192 x 256 outputs per
    block) instead of choosing one, and with ``path`` the kernel that stages tiles through
    "registers" or the one that loads them "direct" into LDS (packed weights, inner size in 64s;
    the only one with shapes 3 and 4)."""
    paths = {None: 0, "registers": 1, "direct": 2, "direct, a block a tile": 3}
    if path not in paths:
        raise ValueError(f"unknown path {path!r}")
    if shape is not None:
        shape = int(shape) + 16 * paths[path]
    before = _hints.tile_shape
    _hints.tile_shape = -1 if shape is None else int(shape)
    try:
        yield
    finally:
        _hints.tile_shape = before


@contextlib.contextmanager
def gemm_few_rows_kernel(which: Optional[str], waves: int = 0, slices: int = 0):
    """For tests and measurements: inside the block this thread's products of up to 64 rows,
    whole or in K slices, go to the kernel ``which`` ("stream", "skinny" or "tiled"; "stream"
    needs packed weights) whatever the sizes, and the stream kernel uses ``waves`` waves per block
    (4 to 8) and aims at ``slices`` K slices (1 to 8); 0: its own choice."""
    if which not in (None, "stream", "skinny", "tiled"):
        raise ValueError(f"unknown kernel {which!r}")
    before = (_hints.few_rows_kernel, _hints.stream)
    _hints.few_rows_kernel = which
    _hints.stream = (int(waves) & 0xff) | ((int(slices) & 0xff) << 8)
    try:
        yield
    finally:
        _hints.few_rows_kernel, _hints.stream = before


MFMA_MAX_HEAD_DIM = 256
# Blocks of four waves that a matrix must give the stream kernel.  A block streams its share of W at
# what one CU pulls, whatever the count of blocks, so fewer blocks than CUs only pay while the
# other kernel, which spreads K over the whole GPU, has more bytes to move than a block's share
# takes: gate/up pairs of 8,960 x 1,536 (140 blocks) 13 to 18 us against 18 to 29 at up to 64 rows,
# 11,008 x 2,048 (172 blocks) 19 to 25 against 25 to 34; 8,192 x 2,048 (128 blocks) 18 against 16,
# and 4,864 x 896 (76 blocks) 4 % slower in a whole decode step.
STREAM_MIN_BLOCKS = 136
STREAM_MIN_BLOCKS_MORE_ROWS = 192        # for 65 to 128 rows
STREAM_MAX_ROWS = 128


def attention_mfma_ok(q_dtype, cache_dtype, head_dim: int) -> bool:
    """Whether the matrix-core attention kernels take these types and this head size."""
    return (q_dtype == torch.bfloat16 and cache_dtype == torch.bfloat16 and head_dim % 16 == 0
            and 16 <= head_dim <= MFMA_MAX_HEAD_DIM)


def attention_decode_mfma(q, k_cache, v_cache, page_table, seq_pos, heads_q, heads_kv, head_dim, scale, window):
    """One bf16 query row per sequence (row i belongs to row i of ``page_table``) at position
    ``seq_pos[i]``, over the cache; keys are split over blocks and merged in ascending order."""
    _dev(q, k_cache, v_cache, page_table, seq_pos)
    n = q.shape[0]
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim or q.dtype != torch.bfloat16:
        raise KernelLibraryError(f"queries must be bfloat16 [sequences, {heads_q * head_dim}]")
    _check_cache(k_cache, v_cache, heads_kv, head_dim)
    _i32(seq_pos, n, "sequence positions")
    if page_table.dtype != torch.int32 or page_table.dim() != 2 or page_table.shape[0] < n:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")
    lib = library.attention_library(head_dim)
    max_pages = page_table.shape[1]
    chunks = lib.sb_attn_decode_chunks(max_pages)
    out = torch.empty_like(q)
    part_o = part_ml = None
    if chunks > 1:
        part_o = torch.empty((lib.sb_attn_decode_part_o(n, heads_q, heads_kv, max_pages),), dtype=torch.float32,
                             device=q.device)
        part_ml = torch.empty((lib.sb_attn_decode_part_ml(n, heads_q, heads_kv, max_pages),), dtype=torch.float32,
                              device=q.device)
    check(lib.sb_attn_decode_bf16(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(page_table), max_pages,
                                  k_cache.shape[0], _p(seq_pos), _p(part_o), _p(part_ml), n, heads_q,
                                  heads_kv, float(scale), int(window), _hints.decode_pages, _stream()),
          lib, "sb_attn_last_error")
    return out


def attention_decode_rope_ok(qkv: torch.Tensor, q_dtype, cache_dtype, heads_q: int, heads_kv: int, head_dim: int,
                             rot_dims: int) -> bool:
    """Whether :func:`attention_decode_rope` takes these operands (else: :func:`rope_kv_store`, then
    :func:`attention`)."""
    if not attention_mfma_ok(q_dtype, cache_dtype, head_dim) or qkv.dtype != torch.float32:
        return False
    lib = library.attention_library(head_dim)
    return bool(lib.sb_attn_decode_rope_ok(heads_q, heads_kv, int(rot_dims), qkv.shape[-1]))


def attention_decode_rope(qkv: torch.Tensor, inv_freq: Optional[torch.Tensor], freq_factors: Optional[torch.Tensor],
                          rot_dims: int, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                          seq_pos: torch.Tensor, heads_q: int, heads_kv: int, head_dim: int, scale: float, window: int,
                          bias: Optional[torch.Tensor] = None, store: bool = True) -> torch.Tensor:
    """A decode step's rotation, store and attention in one kernel: ``qkv`` float32 [n, width] or
    [slices, n, width] (partial sums of the projection, added in ascending order, then ``bias``),
    one row per sequence at position ``seq_pos[i]``.  Queries and keys are rotated as
    :func:`rope_kv_store` rotates them, the row's key and value go into the cache (``store``), and the
    row attends over its sequence's keys, its own among them.  Returns the attention output in
    bfloat16 [n, heads_q * head_dim]: the bits of the two kernels one after the other."""
    _dev(qkv, inv_freq, freq_factors, k_cache, v_cache, page_table, seq_pos, bias)
    n_slices = 1
    if qkv.dim() == 3:
        n_slices = qkv.shape[0]
        qkv = qkv.view(-1, qkv.shape[2])
    n = qkv.shape[0] // n_slices
    need = (heads_q + (2 * heads_kv if store else 0)) * head_dim
    if qkv.dtype != torch.float32 or qkv.shape[1] < need:
        raise KernelLibraryError(f"qkv rows must be float32 with at least {need} elements")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() < need):
        raise KernelLibraryError("the qkv bias must be float32 and cover a whole row")
    if inv_freq is not None:
        if inv_freq.dtype != torch.float32 or inv_freq.numel() != rot_dims // 2:
            raise KernelLibraryError("inv_freq must be float32 [rot_dims/2]")
        if freq_factors is not None and (freq_factors.dtype != torch.float32 or freq_factors.numel() < rot_dims // 2):
            raise KernelLibraryError("freq_factors must be float32 [rot_dims/2]")
    _check_cache(k_cache, v_cache, heads_kv, head_dim)
    if k_cache.dtype != torch.bfloat16:
        raise KernelLibraryError("the fused decode kernel takes a bfloat16 cache")
    _i32(seq_pos, n, "sequence positions")
    if page_table.dtype != torch.int32 or page_table.dim() != 2 or page_table.shape[0] < n:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")
    lib = library.attention_library(head_dim)
    max_pages = page_table.shape[1]
    chunks = lib.sb_attn_decode_chunks(max_pages)
    out = torch.empty((n, heads_q * head_dim), dtype=torch.bfloat16, device=qkv.device)
    part_o = part_ml = None
    if chunks > 1:
        part_o = torch.empty((lib.sb_attn_decode_part_o(n, heads_q, heads_kv, max_pages),), dtype=torch.float32,
                             device=qkv.device)
        part_ml = torch.empty((lib.sb_attn_decode_part_ml(n, heads_q, heads_kv, max_pages),), dtype=torch.float32,
                              device=qkv.device)
    check(lib.sb_attn_decode_rope_bf16(_p(out), _p(qkv), qkv.shape[1], n_slices, _p(bias), _p(inv_freq),
                                       _p(freq_factors), int(rot_dims) if inv_freq is not None else 0,
                                       1 if store else 0, _p(k_cache), _p(v_cache), _p(page_table), max_pages,
                                       k_cache.shape[0], _p(seq_pos), _p(part_o), _p(part_ml), n, heads_q, heads_kv,
                                       float(scale), int(window), _hints.decode_pages, _stream()),
          lib, "sb_attn_last_error")
    return out


@contextlib.contextmanager
def attention_decode_pages_per_wave(head_dim: int, pages: int):
    """For tests and measurements: inside the block this thread's decode attention gives every
    wave ``pages`` pages (1, 2, 4 or 8; more than one only up to head size 128) instead of
    choosing from the sizes; 0: the launcher's choice."""
    before = _hints.decode_pages
    _hints.decode_pages = int(pages)
    try:
        yield
    finally:
        _hints.decode_pages = before


def attention_prefill_mfma(q, k_cache, v_cache, page_table, row_pos, tiles, heads_q, heads_kv, head_dim, scale,
                           window, tile_rows=16):
    """bf16 query rows over the cache; ``tiles`` int32 [n, 4] = (first row, rows <= tile_rows, sequence, 0)
    cuts the rows into runs of consecutive positions of one sequence.  ``tile_rows``: 16, or what
    :func:`attention_row_tile` gives for these heads."""
    _dev(q, k_cache, v_cache, page_table, row_pos, tiles)
    n = q.shape[0]
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim or q.dtype != torch.bfloat16:
        raise KernelLibraryError(f"queries must be bfloat16 [rows, {heads_q * head_dim}]")
    _check_cache(k_cache, v_cache, heads_kv, head_dim)
    _i32(row_pos, n, "row positions")
    if tiles.dtype != torch.int32 or tiles.dim() != 2 or tiles.shape[1] != 4:
        raise KernelLibraryError("tiles must be int32 [n, 4]")
    if page_table.dtype != torch.int32 or page_table.dim() != 2:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")
    lib = library.attention_library(head_dim)
    out = torch.empty_like(q)
    check(lib.sb_attn_prefill_bf16(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(page_table), page_table.shape[1],
                                   k_cache.shape[0], _p(row_pos), _p(tiles), tiles.shape[0], heads_q, heads_kv,
                                   float(scale), int(window), int(tile_rows), _stream()), lib, "sb_attn_last_error")
    return out


# rows of one sequence that a block of the prefill attention kernels takes together; a mixer that
# calls attention() carries it as its row_tile attribute, so that a step describes its rows in
# runs of this height
ATTENTION_ROW_TILE = 16


def attention_row_tile(heads_q: int, heads_kv: int, head_dim: int, dtype=torch.bfloat16) -> int:
    """The height of row tiles that suits attention with these heads: 16, or 64 and 32 where the
    matrix-core kernel runs groups of one and two query heads per kv head (its blocks' waves
    that would have no head take further rows of the tile)."""
    if dtype != torch.bfloat16 or not attention_mfma_ok(dtype, dtype, head_dim) or not torch.cuda.is_available():
        return ATTENTION_ROW_TILE
    return int(library.attention_library(head_dim).sb_attn_prefill_tile_rows(int(heads_q), int(heads_kv)))


# the prefill kernel's second form, for long prompts: tiles of 32 rows (head sizes that 32 divides,
# up to 128, groups of three and more heads); taken when its blocks fill the GPU
TALL_ROW_TILE = 32
TALL_MIN_BLOCKS = 320


def attention_tall_ok(heads_q: int, heads_kv: int, head_dim: int, dtype=torch.bfloat16) -> bool:
    """Whether prefill attention with these heads also runs in tiles of 32 rows."""
    if dtype != torch.bfloat16 or not attention_mfma_ok(dtype, dtype, head_dim) or not torch.cuda.is_available():
        return False
    fn = getattr(library.attention_library(head_dim), "sb_attn_prefill_tall_ok", None)
    return bool(fn is not None and fn(int(heads_q), int(heads_kv)))


def attention_row_tiles(heads_q: int, heads_kv: int, head_dim: int, dtype=torch.bfloat16):
    """The heights of row tiles that a mixer calling :func:`attention` with these heads asks a
    step's context for (its ``row_tile`` attribute): the usual one first."""
    base = attention_row_tile(heads_q, heads_kv, head_dim, dtype)
    if base != TALL_ROW_TILE and attention_tall_ok(heads_q, heads_kv, head_dim, dtype):
        return (base, TALL_ROW_TILE)
    return (base,)


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor, ctx,
              heads_q: int, heads_kv: int, head_dim: int, scale: float, window: int,
              fast: bool = True, row_tile=ATTENTION_ROW_TILE) -> torch.Tensor:
    """Attention of a step's rows over the cache; ``ctx`` is the step's context.  bfloat16 with a
    head size in steps of 16 runs on the matrix cores (a decode kernel when every sequence brings
    one row, else the prefill kernel); everything else takes the plain kernel.  ``row_tile``: the
    height of the context's row tiles to use, or several (what :func:`attention_row_tiles` gives):
    tiles of 32 rows are then taken when their blocks fill the GPU."""
    if fast and attention_mfma_ok(q.dtype, k_cache.dtype, head_dim):
        if ctx.is_decode:
            return attention_decode_mfma(q, k_cache, v_cache, page_table, ctx.row_pos, heads_q, heads_kv,
                                         head_dim, scale, window)
        heights = (row_tile,) if isinstance(row_tile, int) else tuple(row_tile)
        height = heights[0]
        if TALL_ROW_TILE in heights[1:]:
            blocks = ctx.row_tiles(TALL_ROW_TILE).shape[0] * heads_kv * ((heads_q // heads_kv + 7) // 8)
            if blocks >= TALL_MIN_BLOCKS:
                height = TALL_ROW_TILE
        return attention_prefill_mfma(q, k_cache, v_cache, page_table, ctx.row_pos, ctx.row_tiles(height),
                                      heads_q, heads_kv, head_dim, scale, window, tile_rows=height)
    return attention_plain(q, k_cache, v_cache, page_table, ctx.row_pos, ctx.row_seq, heads_q, heads_kv,
                           head_dim, scale, window)


# --------------------------------------------------------------------------
# a gated recurrence; latent attention
# --------------------------------------------------------------------------
def mingru_chunk_rows() -> int:
    """Rows of a chunk of the recurrence's parallel form (the height of the runs of rows it takes)."""
    return int(library.core().sb_mingru_chunk_rows())


def mingru_scan(p: torch.Tensor, state: torch.Tensor, cu_rows: torch.Tensor, slots: torch.Tensor, n_seqs: int,
                out_dtype: torch.dtype, chunks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """minGRU over a step's rows: ``p`` float32 [rows, 3 * width] holds the pre-activations of the
    update gate, the candidate and the output gate; ``state`` float32 [slots, width] is read and
    left moved on for the sequences ``slots`` [n_seqs] whose rows start at ``cu_rows``.  Returns
    S_t * silu(g_t) [rows, width].  ``chunks`` (int32 [n, 4], runs of at most
    :func:`mingru_chunk_rows` rows of one sequence in row order): the parallel form."""
    _dev(p, state, cu_rows, slots, chunks)
    if p.dtype != torch.float32 or p.dim() != 2 or p.shape[1] % 3:
        raise KernelLibraryError("mingru_scan takes float32 rows [rows, 3 * width]")
    rows, width = p.shape[0], p.shape[1] // 3
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != width:
        raise KernelLibraryError(f"the recurrence's state must be float32 [slots, {width}]")
    _i32(cu_rows, n_seqs + 1, "first rows of the sequences")
    _i32(slots, n_seqs, "state rows of the sequences")
    out = torch.empty((rows, width), dtype=out_dtype, device=p.device)
    n_chunks, folded = 0, None
    if chunks is not None:
        if chunks.dtype != torch.int32 or chunks.dim() != 2 or chunks.shape[1] != 4:
            raise KernelLibraryError("chunks must be int32 [n, 4]")
        n_chunks = chunks.shape[0]
        folded = torch.empty((n_chunks, width, 2), dtype=torch.float32, device=p.device)
    check(library.core().sb_mingru_scan(_p(out), _dt(out), _p(p), _p(state), _p(cu_rows), _p(slots), n_seqs, rows,
                                        width, _p(chunks), n_chunks, _p(folded), _stream()))
    return out


def latent_prepare(p: torch.Tensor, q_off: int, kv_off: int, act_dtype: torch.dtype, c_weight: Optional[torch.Tensor],
                   eps: float, inv_freq: Optional[torch.Tensor], rot_dims: int, interleaved: bool,
                   row_pos: torch.Tensor, row_seq: torch.Tensor, cache: Optional[torch.Tensor],
                   page_table: Optional[torch.Tensor], heads: int, dim: int, rot_dim: int, rank: int,
                   kv_rows: Optional[torch.Tensor] = None, magnitude: float = 1.0):
    """``kv_rows`` float32 [rows, m] (a view of rows is fine): the rows that hold the latent's part at
    ``kv_off`` when the queries come out of a product of their own (None: ``p``); ``magnitude``
    multiplies every cosine and sine.  A step's rows of a latent-attention layer's input product ``p`` float32 [rows, n]: returns
    (q_plain [rows, heads, dim], q_latent [rows, heads, rank + rot_dim] whose last rot_dim numbers
    are the rotated query parts; the first rank are left for :func:`head_product`), and, with
    ``kv_off`` >= 0, stores the normed latent and the rotated key part of every row at its
    position in ``cache`` [pages, PAGE, rank + rot_dim]."""
    _dev(p, c_weight, inv_freq, row_pos, row_seq, cache, page_table)
    _on_gpu(kv_rows)
    if p.dtype != torch.float32 or p.dim() != 2:
        raise KernelLibraryError("latent_prepare takes float32 rows")
    n, stride = p.shape
    kv_stride = 0
    if kv_rows is not None:
        if kv_rows.dtype != torch.float32 or kv_rows.dim() != 2 or kv_rows.shape[0] != n or kv_rows.stride(1) != 1 \
                or (kv_off >= 0 and kv_off + rank + rot_dim > kv_rows.shape[1]):
            raise KernelLibraryError("the latent's rows must be float32 [rows, >= kv_off + rank + rot_dim]")
        kv_stride = kv_rows.stride(0) if n > 1 else kv_rows.shape[1]
    latent = rank + rot_dim
    _i32(row_pos, n, "row positions")
    _i32(row_seq, n, "row sequences")
    if rot_dims and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() < rot_dims // 2):
        raise KernelLibraryError("the rotation's table must be float32 with a number per pair")
    max_pages = n_pages = 0
    if kv_off >= 0:
        if cache is None or page_table is None or cache.dim() != 3 or tuple(cache.shape[1:]) != (PAGE, latent):
            raise KernelLibraryError(f"the latent cache must be [pages, {PAGE}, {latent}]")
        if page_table.dtype != torch.int32 or page_table.dim() != 2:
            raise KernelLibraryError("the page table must be int32 [sequences, pages]")
        if c_weight is not None and c_weight.numel() != rank:
            raise KernelLibraryError("the latent's norm weight does not match its size")
        max_pages, n_pages = page_table.shape[1], cache.shape[0]
    q_plain = torch.empty((n, heads, dim), dtype=act_dtype, device=p.device)
    q_latent = torch.empty((n, heads, latent), dtype=act_dtype, device=p.device)
    check(library.core().sb_latent_prepare_split(
        _p(q_plain), _p(q_latent), _DT[act_dtype], _p(p), stride, int(q_off), _p(kv_rows), int(kv_stride), int(kv_off),
        _p(c_weight), _dt(c_weight) if c_weight is not None else 0, float(eps), _p(inv_freq), int(rot_dims),
        1 if interleaved else 0, float(magnitude), _p(row_pos), _p(row_seq), _p(cache) if kv_off >= 0 else None, _dt(cache) if kv_off >= 0 else 0,
        _p(page_table) if kv_off >= 0 else None, max_pages, n_pages, n, heads, dim, rot_dim, rank, _stream()))
    return q_plain, q_latent


def head_product(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None,
                 fast: bool = True, gate_per_head: bool = False) -> torch.Tensor:
    """out[t, a, :n_out] = w[a] x[t, a, :] for every head a: ``x`` [rows, heads, n_in] (a view
    whose last axis is dense), ``w`` [heads, n_out, n_in], ``out`` [rows, heads, >= n_out] (a view
    likewise; only the first n_out numbers of a head are written); ``gate`` float32 [rows, >= heads *
    n_out] (a view of rows): the result times sigmoid(gate); with ``gate_per_head`` the gate is [rows, >= heads],
    one number for all outputs of a head.  bfloat16 operands whose inner size and
    strides are multiples of 8 run on the matrix cores (``fast``), the rest on the plain kernel."""
    for t in (x, w, out, gate):
        if t is not None and not t.is_cuda:
            raise KernelLibraryError("kernel operands must live on the GPU (there is no CPU path)")
    if x.dim() != 3 or w.dim() != 3 or out.dim() != 3 or not w.is_contiguous():
        raise KernelLibraryError("head_product takes x [rows, heads, in], w [heads, out, in], out [rows, heads, out]")
    rows, heads, n_in = x.shape
    n_out = w.shape[1]
    if w.shape[0] != heads or w.shape[2] != n_in or out.shape[0] != rows or out.shape[1] != heads or out.shape[2] < n_out:
        raise KernelLibraryError(f"head_product shapes do not match: x {tuple(x.shape)}, w {tuple(w.shape)}, "
                                 f"out {tuple(out.shape)}")
    if x.stride(2) != 1 or out.stride(2) != 1 or x.dtype != w.dtype:
        raise KernelLibraryError("head_product takes rows that are dense along their last axis, x and w of one type")
    g_stride = 0
    if gate is not None:
        if gate.dtype != torch.float32 or gate.dim() != 2 or gate.shape[0] != rows or gate.stride(1) != 1 \
                or gate.shape[1] < (heads if gate_per_head else heads * n_out):
            raise KernelLibraryError("the gate must be float32 [rows, heads * out] (or [rows, heads], a number a head)")
        g_stride = gate.stride(0)
    lib = library.core()
    if fast and x.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and x.data_ptr() % 16 == 0 \
            and w.data_ptr() % 16 == 0 and lib.sb_head_product_bf16_ok(out.stride(0), out.stride(1), x.stride(0),
                                                                       x.stride(1), n_in):
        check(lib.sb_head_product_gated_bf16(_p(out), out.stride(0), out.stride(1), _p(x), x.stride(0), x.stride(1), _p(w),
                                             _p(gate), g_stride, 1 if gate_per_head else 0, rows, heads, n_in, n_out,
                                             _stream()))
        return out
    check(lib.sb_head_product_gated(_p(out), _dt(out), out.stride(0), out.stride(1), _p(x), _dt(x), x.stride(0),
                                    x.stride(1), _p(w), _dt(w), _p(gate), g_stride, 1 if gate_per_head else 0, rows, heads,
                                    n_in, n_out, _stream()))
    return out


def latent_attention_plain(q: torch.Tensor, cache: torch.Tensor, page_table: torch.Tensor, row_pos: torch.Tensor,
                           row_seq: torch.Tensor, rank: int, scale: float, window: int) -> torch.Tensor:
    """Softmax attention of ``q`` [rows, heads, latent] over the cached rows [pages, PAGE, latent]
    each row sees; returns the weighted sums of the rows' first ``rank`` numbers [rows, heads, rank]."""
    _dev(q, cache, page_table, row_pos, row_seq)
    if q.dim() != 3 or cache.dim() != 3 or cache.shape[1] != PAGE or cache.shape[2] != q.shape[2]:
        raise KernelLibraryError("latent attention takes q [rows, heads, latent] and a cache [pages, PAGE, latent]")
    n, heads, latent = q.shape
    _i32(row_pos, n, "row positions")
    _i32(row_seq, n, "row sequences")
    if page_table.dtype != torch.int32 or page_table.dim() != 2:
        raise KernelLibraryError("the page table must be int32 [sequences, pages]")
    out = torch.empty((n, heads, rank), dtype=q.dtype, device=q.device)
    check(library.core().sb_latent_attention(_p(out), _p(q), _dt(q), _p(cache), _dt(cache), _p(page_table),
                                             page_table.shape[1], cache.shape[0], _p(row_pos), _p(row_seq), n, heads,
                                             rank, latent - rank, float(scale), int(window), _stream()))
    return out


LATENT_ROW_TILE = 16        # rows of a run that a prompt step's matrix-core launch takes (sb_latent_attention_tile_rows)


def latent_attention_mfma_ok(q_dtype, cache_dtype, rank: int, rot_dim: int) -> bool:
    return q_dtype == torch.bfloat16 and cache_dtype == torch.bfloat16 \
        and bool(library.core().sb_latent_attention_bf16_ok(int(rank), int(rot_dim)))


LATENT_SPLIT_BLOCKS = 512       # blocks a step of few rows aims at by sharing out its keys
LATENT_SPLIT_KEYS = 128         # keys a share has at least (64: 45 us, 128: 41, 256: 50 for 8 rows over 2,049 keys of 576 numbers)


def latent_attention_mfma(q: torch.Tensor, cache: torch.Tensor, page_table: torch.Tensor, row_pos: torch.Tensor,
                          tiles: torch.Tensor, rank: int, scale: float, window: int, single_rows: bool,
                          max_keys: int = 0) -> torch.Tensor:
    """The matrix-core form: ``tiles`` int32 [n, 4], runs of up to 16 consecutive rows of a sequence;
    ``single_rows``: every run is one row (a decode step), a wave then takes 16 heads of it.
    ``max_keys`` (the most keys a row of the step sees, if the caller knows): a launch of few blocks
    over many keys shares the keys of every run out over several blocks and merges their results."""
    _dev(q, cache, page_table, row_pos, tiles)
    n, heads, latent = q.shape
    if cache.dim() != 3 or cache.shape[1] != PAGE or cache.shape[2] != latent:
        raise KernelLibraryError("latent attention takes q [rows, heads, latent] and a cache [pages, PAGE, latent]")
    _i32(row_pos, n, "row positions")
    if tiles.dtype != torch.int32 or tiles.dim() != 2 or tiles.shape[1] != 4:
        raise KernelLibraryError("row tiles must be int32 [n, 4]")
    if page_table.dtype != torch.int32 or page_table.dim() != 2:
        raise KernelLibraryError("the page table must be int32 [sequences, pages]")
    out = torch.empty((n, heads, rank), dtype=q.dtype, device=q.device)
    blocks = tiles.shape[0] * -(-heads // (64 if single_rows else 4))
    splits = 1
    if max_keys > LATENT_SPLIT_KEYS and 0 < blocks < LATENT_SPLIT_BLOCKS:
        splits = max(1, min(-(-LATENT_SPLIT_BLOCKS // blocks), max_keys // LATENT_SPLIT_KEYS))
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty((splits, n, heads, rank), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((splits, n, heads, 2), dtype=torch.float32, device=q.device)
    check(library.core().sb_latent_attention_bf16(_p(out), _p(q), _p(cache), _p(page_table), page_table.shape[1],
                                                  cache.shape[0], _p(row_pos), _p(tiles), tiles.shape[0], heads, rank,
                                                  latent - rank, float(scale), int(window), 1 if single_rows else 16,
                                                  splits, _p(part_o), _p(part_ml), n, _stream()))
    return out


def latent_attention(q: torch.Tensor, cache: torch.Tensor, page_table: torch.Tensor, ctx, rank: int, scale: float,
                     window: int, fast: bool = True) -> torch.Tensor:
    """Latent attention of a step's rows: the matrix-core kernel where it takes the sizes and
    types (the step's context then lists the rows in runs of LATENT_ROW_TILE), else the kernel of
    one wave per (row, head)."""
    if fast and latent_attention_mfma_ok(q.dtype, cache.dtype, rank, q.shape[2] - rank):
        keys = int(getattr(ctx, "max_len_after", 0) or 0)
        return latent_attention_mfma(q, cache, page_table, ctx.row_pos, ctx.row_tiles(LATENT_ROW_TILE), rank, scale,
                                     window, single_rows=bool(ctx.is_decode),
                                     max_keys=min(keys, window) if window > 0 else keys)
    return latent_attention_plain(q, cache, page_table, ctx.row_pos, ctx.row_seq, rank, scale, window)


# --------------------------------------------------------------------------
# norms of what leaves a sublayer; an embedding with positions; head norms; capped attention; experts
# --------------------------------------------------------------------------
def offset_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, offset: float, out_dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * (offset + weight) of float32 rows ``x`` [n, width]; ``rows``
    (int32) picks and orders source rows."""
    _dev(x, weight, rows)
    if x.dtype != torch.float32 or x.dim() != 2:
        raise KernelLibraryError("the norm's input must be float32 [rows, width]")
    width = x.shape[1]
    if weight is not None and weight.numel() != width:
        raise KernelLibraryError(f"the norm's weight has {weight.numel()} elements, the rows have {width}")
    n = x.shape[0] if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, n, "row index")
    y = torch.empty((n, width), dtype=out_dtype, device=x.device)
    check(library.core().sb_offset_norm(_p(y), _dt(y), _p(x), _p(weight), _dt(weight) if weight is not None else 0,
                                        _p(rows), n, width, float(eps), float(offset), _stream()))
    return y


def norm_add(x: torch.Tensor, part: torch.Tensor, weight: Optional[torch.Tensor], eps: float, offset: float,
             copy_dtype: Optional[torch.dtype] = None, part_weights: Optional[torch.Tensor] = None,
             extra: Optional[torch.Tensor] = None, extra_weights: Optional[torch.Tensor] = None,
             by_row: bool = False, norm: bool = True) -> Optional[torch.Tensor]:
    """x += un(sum_s a_s part_s (+ b extra)), un(v) = v / sqrt(mean(v^2) + eps) * (offset + weight)
    (``norm`` false: the sum as it is); returns the new x in ``copy_dtype`` when that is given.

    ``part`` float32 [rows, width], or slices of it: [slices, rows, width], or with ``by_row``
    [rows, slices, width].  ``part_weights`` (float32, a view [rows, slices] of rows that may be
    longer): the multiplier a_s of every row's slices, else 1.  ``extra`` float32 [rows, width] with
    ``extra_weights`` (a view [rows] or [rows, 1]) one multiplier a row."""
    _dev(x, part, weight, extra)
    if x.dtype != torch.float32 or x.dim() != 2:
        raise KernelLibraryError("the stream must be float32 [rows, width]")
    n, width = x.shape
    if part.dtype != torch.float32:
        raise KernelLibraryError("the sublayer's result must be float32")
    if part.dim() == 2:
        part = part.view(1, n, width)
        by_row = False
    if part.dim() != 3 or part.shape[2] != width or part.shape[0 if by_row else 1] != n:
        raise KernelLibraryError(f"the sublayer's result {tuple(part.shape)} does not fit the stream {tuple(x.shape)}")
    slices = part.shape[1 if by_row else 0]
    slice_stride, row_stride = (width, slices * width) if by_row else (n * width, width)
    pw_stride = ew_stride = 0
    for t, what in ((part_weights, "slice"), (extra_weights, "row")):
        if t is not None and (t.dtype != torch.float32 or not t.is_cuda or t.shape[0] != n or t.stride(-1) != 1):
            raise KernelLibraryError(f"the {what} multipliers must be float32 rows on the GPU")
    if part_weights is not None:
        if part_weights.dim() != 2 or part_weights.shape[1] != slices:
            raise KernelLibraryError("one multiplier for every slice of every row")
        pw_stride = part_weights.stride(0)
    if extra is not None:
        if extra.dtype != torch.float32 or tuple(extra.shape) != (n, width):
            raise KernelLibraryError("the extra addend must be float32 and shaped like the stream")
        if extra_weights is not None:
            ew_stride = extra_weights.stride(0)
    if weight is not None and weight.numel() != width:
        raise KernelLibraryError(f"the norm's weight has {weight.numel()} elements, the rows have {width}")
    copy = None
    if copy_dtype is not None and copy_dtype != torch.float32:
        copy = torch.empty((n, width), dtype=copy_dtype, device=x.device)
    check(library.core().sb_norm_add(
        _p(x), _p(copy), _dt(copy) if copy is not None else 0, _p(part), slices, slice_stride, row_stride,
        _p(part_weights), pw_stride, _p(extra), _p(extra_weights) if extra is not None else None, ew_stride,
        _p(weight), _dt(weight) if weight is not None else 0, n, width, float(eps), float(offset), 1 if norm else 0,
        _stream()))
    return x if copy_dtype == torch.float32 else copy


def embed_pos_norm(table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0, positions: Optional[torch.Tensor] = None,
                   row_pos: Optional[torch.Tensor] = None, weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                   offset: float = 0.0, norm: bool = False, copy_dtype: Optional[torch.dtype] = None):
    """x = table[ids] * scale (+ positions[row_pos]), then with ``norm`` x / sqrt(mean(x^2) + eps) *
    (offset + weight); float32 [n, width], and a copy in ``copy_dtype`` when that is given (and not
    float32).  An id or a position outside its table gives a row of NaN."""
    _dev(table, ids, positions, row_pos, weight)
    if table.dim() != 2 or (positions is not None and (positions.dim() != 2 or positions.shape[1] != table.shape[1])):
        raise KernelLibraryError("the tables must be [vocab, width] and [positions, width]")
    n = ids.numel()
    _i32(ids, n, "token ids")
    if positions is not None:
        if row_pos is None:
            raise KernelLibraryError("a table of positions needs the rows' positions")
        _i32(row_pos, n, "row positions")
    vocab, width = table.shape
    if weight is not None and weight.numel() != width:
        raise KernelLibraryError(f"the norm's weight has {weight.numel()} elements, the rows have {width}")
    x = torch.empty((n, width), dtype=torch.float32, device=table.device)
    copy = None
    if copy_dtype is not None and copy_dtype != torch.float32:
        copy = torch.empty((n, width), dtype=copy_dtype, device=table.device)
    check(library.core().sb_embed_pos_norm(
        _p(x), _p(copy), _dt(copy) if copy is not None else 0, _p(table), _dt(table), _p(positions),
        _dt(positions) if positions is not None else 0, _p(ids), _p(row_pos), n, vocab,
        positions.shape[0] if positions is not None else 0, float(scale), _p(weight),
        _dt(weight) if weight is not None else 0, width, float(eps), float(offset), 1 if norm else 0, _stream()))
    return x, copy


def _check_cache_kv(k_cache, v_cache, heads_kv, head_dim, v_dim):
    if k_cache.dim() != 4 or v_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (heads_kv, PAGE, head_dim) \
            or tuple(v_cache.shape[1:]) != (heads_kv, v_dim, PAGE) or k_cache.shape[0] != v_cache.shape[0] \
            or k_cache.dtype != v_cache.dtype:
        raise KernelLibraryError(
            f"cache must be keys [pages, {heads_kv}, {PAGE}, {head_dim}] and values "
            f"[pages, {heads_kv}, {v_dim}, {PAGE}], found {tuple(k_cache.shape)} and {tuple(v_cache.shape)}")


def headnorm_kv_store(qkv: torch.Tensor, q_dtype: torch.dtype, q_weight: Optional[torch.Tensor],
                      k_weight: Optional[torch.Tensor], eps: float, row_pos: torch.Tensor, row_seq: torch.Tensor,
                      k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
                      heads_q: int, heads_kv: int, head_dim: int, v_dim: int, store: bool = True,
                      v_first: Optional[torch.Tensor] = None, lam: Optional[torch.Tensor] = None,
                      v_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From float32 rows [n, heads_q*head_dim + heads_kv*(head_dim + v_dim)] of a stacked product (or
    [slices, n, ...], added here): every head of q and k divided by its root mean square and
    multiplied by a weight [head_dim] that the heads share (None: as it is), the values mixed as
    (1 - lam) v + lam v_first when ``v_first`` (float32 [n, heads_kv*v_dim]) is given, the values of
    before the mixing written to ``v_out``; returns q [n, heads_q*head_dim] in ``q_dtype`` and, with
    ``store``, puts keys and values into the pages of the rows' positions."""
    _dev(qkv, q_weight, k_weight, row_pos, row_seq, k_cache, v_cache, page_table, v_first, lam, v_out)
    if qkv.dtype != torch.float32:
        raise KernelLibraryError("the stacked product must be float32")
    n_slices = 1
    if qkv.dim() == 3:
        n_slices = qkv.shape[0]
        qkv = qkv.view(-1, qkv.shape[2])
    n = qkv.shape[0] // n_slices
    need = heads_q * head_dim + (heads_kv * (head_dim + v_dim) if store else 0)
    if qkv.dim() != 2 or qkv.shape[1] < need:
        raise KernelLibraryError(f"rows of the stacked product have {qkv.shape[1]} elements, {need} are needed")
    for w in (q_weight, k_weight):
        if w is not None and w.numel() != head_dim:
            raise KernelLibraryError(f"a head norm's weight has {w.numel()} elements, a head has {head_dim}")
    if q_weight is not None and k_weight is not None and q_weight.dtype != k_weight.dtype:
        raise KernelLibraryError("the head norms' weights must be of one type")
    wt = q_weight if q_weight is not None else k_weight
    max_pages = n_pages = 0
    if store:
        _check_cache_kv(k_cache, v_cache, heads_kv, head_dim, v_dim)
        _check_rows(row_pos, row_seq, page_table, n)
        max_pages, n_pages = page_table.shape[1], k_cache.shape[0]
    nv = heads_kv * v_dim
    for t, what in ((v_first, "values to mix with"), (v_out, "values to hand on")):
        if t is not None and (t.dtype != torch.float32 or t.numel() != n * nv):
            raise KernelLibraryError(f"the {what} must be float32 [rows, {nv}]")
    if v_first is not None and (lam is None or lam.numel() != 1):
        raise KernelLibraryError("mixing values takes one number")
    q = torch.empty((n, heads_q * head_dim), dtype=q_dtype, device=qkv.device)
    check(library.core().sb_headnorm_kv_store(
        _p(q), _dt(q), _p(qkv), qkv.shape[1], n_slices, _p(q_weight), _p(k_weight), _dt(wt) if wt is not None else 0,
        float(eps), _p(v_first), _p(lam) if v_first is not None else None, _dt(lam) if lam is not None else 0, _p(v_out),
        _p(row_pos), _p(row_seq), _p(k_cache), _p(v_cache), _dt(k_cache) if store else 0, _p(page_table), max_pages,
        n_pages, n, heads_q, heads_kv, head_dim, v_dim, 1 if store else 0, _stream()))
    return q


def attention_capped_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                           row_pos: torch.Tensor, row_seq: torch.Tensor, heads_q: int, heads_kv: int, head_dim: int,
                           v_dim: int, scale: float, window: int, softcap: float, sink: bool,
                           sink_scores: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of rows ``q`` [n, hq*hd] over the cache by the plain kernel, values of ``v_dim``,
    scores capped as softcap tanh(s / softcap) (0: not), with ``sink`` one more key of score 0
    without a value in every softmax (``sink_scores`` float32 [hq]: of the head's own score instead); [n, hq*v_dim].
    ``gate`` float32 [n, hq*v_dim] (a view of wider rows is fine): the result times sigmoid(gate)."""
    _dev(q, k_cache, v_cache, page_table, row_pos, row_seq, sink_scores)
    _check_sink(sink, sink_scores, heads_q)
    g_stride = _check_gate(gate, q.shape[0], heads_q * v_dim)
    n = q.shape[0]
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim:
        raise KernelLibraryError(f"queries must be [rows, {heads_q * head_dim}]")
    _check_cache_kv(k_cache, v_cache, heads_kv, head_dim, v_dim)
    _check_rows(row_pos, row_seq, page_table, n)
    out = torch.empty((n, heads_q * v_dim), dtype=q.dtype, device=q.device)
    check(library.core().sb_attention_sink(
        _p(out), _p(q), _dt(q), q.shape[1], _p(k_cache), _p(v_cache), _dt(k_cache), _p(page_table),
        page_table.shape[1], k_cache.shape[0], _p(row_pos), _p(row_seq), n, heads_q, heads_kv, head_dim, v_dim,
        float(scale), int(window), float(softcap), 1 if sink else 0, _p(sink_scores), _p(gate), g_stride, _stream()))
    return out


def _check_gate(gate, rows, width) -> int:
    """The distance between the rows of an output gate (0 without one)."""
    if gate is None:
        return 0
    _on_gpu(gate)
    if gate.dtype != torch.float32 or gate.dim() != 2 or tuple(gate.shape) != (rows, width) or gate.stride(1) != 1:
        raise KernelLibraryError(f"an output gate must be float32 [{rows}, {width}], dense along a row")
    return gate.stride(0) if rows > 1 else width


def _check_sink(sink, sink_scores, heads_q):
    if sink_scores is not None and (not sink or sink_scores.dtype != torch.float32 or sink_scores.numel() != heads_q
                                    or not sink_scores.is_contiguous()):
        raise KernelLibraryError(f"a sink's scores must be float32 [{heads_q}], of a sink that is switched on")


def scale_(x: torch.Tensor, scale: float) -> torch.Tensor:
    """x *= scale in place (float32)."""
    _dev(x)
    if x.dtype != torch.float32:
        raise KernelLibraryError("scale_ takes float32 values")
    check(library.core().sb_scale(_p(x), float(scale), x.numel(), _stream()))
    return x


MOE_MAX_TOP = 16        # choices a row that the router kernel takes (sb_moe_max_top)


class MoEWeight:
    """The stacked matrices of a set of experts, [experts, out (or 2 * out: gate over up), in], as
    the experts' product kernels read them."""

    def __init__(self, w: torch.Tensor, gated: bool = False, fast: bool = True):
        if w.dim() != 3 or (gated and w.shape[1] % 2):
            raise KernelLibraryError("experts' matrices must be stacked [experts, out, in]")
        self.w = w.contiguous()
        self.gated = gated
        self.experts, rows, self.n_in = w.shape
        self.n_out = rows // 2 if gated else rows
        self.fast = fast


class MoEPlan:
    """Which expert every (row, choice) pair takes: ``ids`` int32 [pairs] (None: all take expert 0),
    and, once :meth:`group` has run, the pairs laid out expert by expert for the matrix-core product:
    ``order`` int32 [pairs], ``tiles`` int32 [max_tiles, 4] = (expert, first place in order, pairs, 0),
    ``n_tiles`` int32 [1] on the device."""

    def __init__(self, ids: Optional[torch.Tensor], n_pairs: int, n_experts: int):
        self.ids, self.n_pairs, self.n_experts = ids, n_pairs, n_experts
        self.tile_rows = int(library.core().sb_moe_tile_rows(n_pairs, n_experts)) if n_pairs else 64
        self.order = self.tiles = self.n_tiles = None
        self.max_tiles = 0

    def group(self) -> None:
        if self.ids is None or self.order is not None or self.n_pairs == 0:
            return
        dev = self.ids.device
        self.max_tiles = self.n_pairs // self.tile_rows + self.n_experts + 1
        self.order = torch.empty(self.n_pairs, dtype=torch.int32, device=dev)
        self.tiles = torch.empty((self.max_tiles, 4), dtype=torch.int32, device=dev)
        self.n_tiles = torch.empty(1, dtype=torch.int32, device=dev)
        check(library.core().sb_moe_group(_p(self.ids), self.n_pairs, self.n_experts, self.tile_rows, _p(self.order),
                                          _p(self.tiles), _p(self.n_tiles), _stream()))


def moe_plan(ids: Optional[torch.Tensor], n_experts: int, n_pairs: Optional[int] = None, device=None) -> MoEPlan:
    if ids is not None:
        _dev(ids)
        ids = ids.view(-1)
        _i32(ids, ids.numel(), "expert numbers")
        n_pairs = ids.numel()
    return MoEPlan(ids, int(n_pairs), int(n_experts))


def _expert_code(gated: bool, pair: str, single: Optional[str]) -> int:
    """The `gated` argument of the experts' products."""
    if gated:
        if single is not None:
            raise KernelLibraryError("a gated weight gives pairs; an activation of its own belongs to experts without a gate")
        return EXPERT_PAIRS[pair]
    return EXPERT_SINGLES[single] if single is not None else 0


def moe_product(x: torch.Tensor, w: MoEWeight, plan: MoEPlan, x_div: int, out_dtype: torch.dtype,
                limit: float = 0.0, alpha: float = 1.0, pair: str = "swish_clamp", single: Optional[str] = None) -> torch.Tensor:
    """Y[p] = X[p // x_div] W_e^T for every pair p of ``plan``; a gated weight gives the pair of its
    two halves that ``pair`` names (the clamped swish pair, or "silu": silu(g) u); a weight without a gate
    takes ``single``, the activation of every output ("relu_sq": max(z, 0)^2; None: the product as it is).  bfloat16 operands with an inner size in eights run on the matrix
    cores, the pairs grouped by expert on the device; everything else takes the plain kernel."""
    if w.experts != plan.n_experts:
        raise KernelLibraryError(f"the plan counts {plan.n_experts} experts, the weight has {w.experts}")
    if not (w.fast and x.dtype == torch.bfloat16 and w.w.dtype == torch.bfloat16 and w.n_in % 8 == 0):
        return moe_product_plain(x, w.w, plan.ids, plan.n_pairs, x_div, out_dtype, w.gated, limit, alpha, pair, single)
    _dev(x)
    if x.dim() != 2 or x.shape[1] != w.n_in or (plan.n_pairs + x_div - 1) // x_div > x.shape[0]:
        raise KernelLibraryError(f"expert product shapes do not match: x {tuple(x.shape)}, w {tuple(w.w.shape)}, "
                                 f"{plan.n_pairs} pairs")
    plan.group()
    y = torch.empty((plan.n_pairs, w.n_out), dtype=out_dtype, device=x.device)
    check(library.core().sb_moe_product_bf16(
        _p(y), _dt(y), _p(x), _p(w.w), _p(plan.order), _p(plan.tiles), _p(plan.n_tiles), plan.max_tiles, plan.tile_rows,
        plan.n_pairs, int(x_div), w.n_out, w.n_in, _expert_code(w.gated, pair, single), float(limit), float(alpha), _stream()))
    return y


def attention_capped(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor, ctx,
                     heads_q: int, heads_kv: int, head_dim: int, v_dim: int, scale: float, window: int,
                     softcap: float, sink: bool, fast: bool = True, sink_scores: Optional[torch.Tensor] = None,
                     gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of a step's rows over the cache with values of their own size, capped scores and a
    sink (see :func:`attention_capped_plain`).  bfloat16 with key and value sizes in steps of 16
    runs on the matrix cores; everything else takes the plain kernel."""
    if fast and capped_attention_mfma_ok(q.dtype, k_cache.dtype, head_dim, v_dim):
        return attention_capped_mfma(q, k_cache, v_cache, page_table, ctx.row_pos, ctx.row_tiles(CAPPED_ROW_TILE),
                                     heads_q, heads_kv, head_dim, v_dim, scale, window, softcap, sink,
                                     sink_scores=sink_scores, gate=gate)
    return attention_capped_plain(q, k_cache, v_cache, page_table, ctx.row_pos, ctx.row_seq, heads_q, heads_kv,
                                  head_dim, v_dim, scale, window, softcap, sink, sink_scores, gate)


CAPPED_ROW_TILE = 16        # rows of a run that a block of the matrix-core kernel takes (sb_cattn_tile_rows)
CAPPED_SPLIT_BLOCKS = 512   # blocks a step of few rows aims at by sharing out its pages


def capped_attention_mfma_ok(q_dtype, cache_dtype, head_dim: int, v_dim: int) -> bool:
    return (q_dtype == torch.bfloat16 and cache_dtype == torch.bfloat16
            and all(n % 16 == 0 and 16 <= n <= MFMA_MAX_HEAD_DIM for n in (head_dim, v_dim)))


def attention_capped_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                          row_pos: torch.Tensor, tiles: torch.Tensor, heads_q: int, heads_kv: int, head_dim: int,
                          v_dim: int, scale: float, window: int, softcap: float, sink: bool,
                          chunks: Optional[int] = None, sink_scores: Optional[torch.Tensor] = None,
                          gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The matrix-core form of :func:`attention_capped_plain`.  ``tiles`` int32 [n, 4]: the rows in
    runs of up to 16 consecutive rows of one sequence.  ``chunks``: over how many blocks a run's
    pages are shared out (None: chosen from the shapes alone, so that a recorded step replays)."""
    _dev(q, k_cache, v_cache, page_table, row_pos, tiles, sink_scores)
    _check_sink(sink, sink_scores, heads_q)
    n = q.shape[0]
    g_stride = _check_gate(gate, n, heads_q * v_dim)
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim or q.dtype != torch.bfloat16:
        raise KernelLibraryError(f"queries must be bfloat16 [rows, {heads_q * head_dim}]")
    _check_cache_kv(k_cache, v_cache, heads_kv, head_dim, v_dim)
    if k_cache.dtype != torch.bfloat16:
        raise KernelLibraryError("the matrix-core kernel reads a bfloat16 cache")
    _i32(row_pos, n, "row positions")
    if page_table.dtype != torch.int32 or page_table.dim() != 2:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")
    if tiles.dtype != torch.int32 or tiles.dim() != 2 or tiles.shape[1] != 4:
        raise KernelLibraryError("row tiles must be int32 [n, 4]")
    n_tiles, max_pages = tiles.shape[0], page_table.shape[1]
    group = heads_q // heads_kv
    blocks = max(1, n_tiles * heads_kv * ((group + 3) // 4))
    if chunks is None:
        chunks = max(1, min(max_pages, CAPPED_SPLIT_BLOCKS // blocks))
    chunk_pages = (max_pages + chunks - 1) // chunks
    chunks = (max_pages + chunk_pages - 1) // chunk_pages
    part_o = part_ml = None
    if chunks > 1:
        part_o = torch.empty((chunks, n, heads_q, v_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((chunks, n, heads_q, 2), dtype=torch.float32, device=q.device)
    out = torch.empty((n, heads_q * v_dim), dtype=torch.bfloat16, device=q.device)
    lib = library.capped_attention_library(head_dim, v_dim)
    check(lib.sb_cattn_sink_bf16(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(page_table), max_pages, k_cache.shape[0],
                                 _p(row_pos), _p(tiles), n_tiles, n, heads_q, heads_kv, float(scale), int(window),
                                 float(softcap), 1 if sink else 0, chunks, chunk_pages, _p(part_o), _p(part_ml), None, None, 0,
                                 _p(sink_scores), _p(gate), g_stride, _stream()),
          lib, "sb_cattn_last_error")
    return out


def moe_max_top() -> int:
    return int(library.core().sb_moe_max_top())


def moe_route(z: torch.Tensor, n_experts: int, top: int, has_gate: bool, score: str = "softmax_chosen", score_scale: float = 1.0,
              groups: int = 1, keep_groups: int = 1):
    """From router scores ``z`` float32 [n, >= n_experts (+ 1)]: the ``top`` largest of the first
    ``n_experts`` of every row (ties to the lower number) as int32 [n, top], and float32 [n, top + 1]:
    the softmax over the chosen scores, then sigmoid(z[:, n_experts]) with ``has_gate`` (else 0).
    ``score`` "sigmoid": the scores are sigmoid(z), the largest are chosen and their weights are those
    scores times ``score_scale``, not renormalized; "softmax_all": the same with the softmax of z over
    all experts as scores.  ``groups`` > 1: the experts lie in that many equal groups of neighbours, a
    group's score is its best expert's, and only experts of the ``keep_groups`` best groups are chosen."""
    _dev(z)
    if z.dtype != torch.float32 or z.dim() != 2:
        raise KernelLibraryError("router scores must be float32 [rows, experts]")
    n = z.shape[0]
    ids = torch.empty((n, top), dtype=torch.int32, device=z.device)
    weights = torch.empty((n, top + 1), dtype=torch.float32, device=z.device)
    check(library.core().sb_moe_route_grouped(_p(ids), _p(weights), _p(z), n, z.shape[1], int(n_experts), int(top),
                                              1 if has_gate else 0, ROUTER_SCORES[score], float(score_scale), int(groups),
                                              int(keep_groups), _stream()))
    return ids, weights


def moe_router(h: torch.Tensor, w: torch.Tensor, n_experts: int, top: int, has_gate: bool, score: str = "softmax_chosen",
               score_scale: float = 1.0, groups: int = 1, keep_groups: int = 1):
    """The router in one launch: z = h w^T in float32 (``w`` float32 [n_experts (+ 1 with
    ``has_gate``), width], ``h`` rows of either type), then what :func:`moe_route` gives."""
    _dev(h, w)
    if w.dtype != torch.float32 or w.dim() != 2 or h.dim() != 2 or h.shape[1] != w.shape[1] \
            or w.shape[0] != n_experts + (1 if has_gate else 0):
        raise KernelLibraryError(f"the router's matrix must be float32 [{n_experts + (1 if has_gate else 0)}, {h.shape[-1]}]")
    n = h.shape[0]
    ids = torch.empty((n, top), dtype=torch.int32, device=h.device)
    weights = torch.empty((n, top + 1), dtype=torch.float32, device=h.device)
    check(library.core().sb_moe_router_grouped(_p(ids), _p(weights), _p(h), _dt(h), _p(w), n, h.shape[1], int(n_experts),
                                               int(top), 1 if has_gate else 0, ROUTER_SCORES[score], float(score_scale),
                                               int(groups), int(keep_groups), _stream()))
    return ids, weights


def swish_clamp_mul(gu: torch.Tensor, out_dtype: torch.dtype, limit: float, alpha: float) -> torch.Tensor:
    """g' sigmoid(alpha g') (u' + 1) for gu = [g | u] float32 [n, 2w], g' = min(g, limit), u' = u cut to +-limit."""
    _dev(gu)
    if gu.dtype != torch.float32 or gu.dim() != 2 or gu.shape[1] % 2:
        raise KernelLibraryError("the pair's input must be float32 [rows, 2*width]")
    n, w2 = gu.shape
    out = torch.empty((n, w2 // 2), dtype=out_dtype, device=gu.device)
    check(library.core().sb_swish_clamp_mul(_p(out), _dt(out), _p(gu), n, w2 // 2, float(limit), float(alpha), _stream()))
    return out


def moe_product_plain(x: torch.Tensor, w: torch.Tensor, ids: Optional[torch.Tensor], n_pairs: int, x_div: int,
                      out_dtype: torch.dtype, gated: bool = False, limit: float = 0.0, alpha: float = 1.0,
                      pair: str = "swish_clamp", single: Optional[str] = None) -> torch.Tensor:
    """Y[p] = X[p // x_div] W_e^T, e = ids[p] (None: expert 0), by the plain kernel.  ``w``
    [experts, out (or 2*out, gate over up, with ``gated``), in]; gated: the clamped swish pair
    g' sigmoid(alpha g') (u' + 1) with g' = min(g, limit), u' = u cut to +-limit."""
    _dev(x, w, ids)
    if w.dim() != 3 or x.dim() != 2 or x.shape[1] != w.shape[2]:
        raise KernelLibraryError(f"expert product shapes do not match: x {tuple(x.shape)}, w {tuple(w.shape)}")
    n_experts, rows, n_in = w.shape
    n_out = rows // 2 if gated else rows
    if ids is not None:
        _i32(ids, n_pairs, "expert numbers")
    if (n_pairs + x_div - 1) // x_div > x.shape[0]:
        raise KernelLibraryError("more pairs than rows to take them from")
    y = torch.empty((n_pairs, n_out), dtype=out_dtype, device=x.device)
    check(library.core().sb_moe_product(_p(y), _dt(y), _p(x), _dt(x), _p(w), _dt(w), _p(ids), n_pairs, int(x_div),
                                        n_out, n_in, n_experts, _expert_code(gated, pair, single), float(limit), float(alpha),
                                        _stream()))
    return y


# ---- short convolutions over time, recurrences with a matrix state, attention with shared weights ----
ROUTER_SCORES = {"softmax_chosen": 0, "sigmoid": 1, "softmax_all": 2}      # score_kind of sb_moe_route_grouped
EXPERT_PAIRS = {"swish_clamp": 1, "silu": 2}             # `gated` of the experts' products: pairs of a gate and an up row
EXPERT_SINGLES = {"relu_sq": 3}                          # the same argument for experts without a gate: one row an output


def time_conv_max_taps() -> int:
    return int(library.core().sb_time_conv_max_taps())


def time_conv(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, ctx,
              out_dtype: torch.dtype, activation: Optional[str] = None, residual: bool = False,
              columns: Optional[tuple] = None) -> torch.Tensor:
    """y[t] = act(sum_j weight[:, j] x[t - taps + 1 + j] (+ bias)) (+ x[t] with ``residual``), channel by
    channel over the rows of every sequence of the step ``ctx``; the rows before a step's first are
    the sequence's ``state`` float32 [slots, taps - 1, channels], which is moved on.  ``columns``
    (first, count): the channels are that range of the columns of ``x``.  ``activation``: None or "silu"."""
    _dev(x, weight, bias, state)
    if x.dim() != 2 or weight.dim() != 2:
        raise KernelLibraryError("the convolution takes rows [n, columns] and taps [channels, taps]")
    first, channels = columns if columns is not None else (0, x.shape[1])
    taps = weight.shape[1]
    if weight.shape[0] != channels or first < 0 or first + channels > x.shape[1]:
        raise KernelLibraryError(f"taps {tuple(weight.shape)} do not fit {channels} channels from column {first} of {x.shape[1]}")
    if bias is not None and bias.numel() != channels:
        raise KernelLibraryError(f"the bias has {bias.numel()} elements for {channels} channels")
    if state.dtype != torch.float32 or state.dim() != 3 or tuple(state.shape[1:]) != (taps - 1, channels):
        raise KernelLibraryError(f"the state must be float32 [slots, {taps - 1}, {channels}], not {tuple(state.shape)}")
    if activation not in (None, "silu"):
        raise KernelLibraryError(f"the convolution's activation is None or 'silu', not {activation!r}")
    n = x.shape[0]
    if n != ctx.n_rows:
        raise KernelLibraryError("the rows are not those of the step")
    _i32(ctx.row_seq, n, "row sequences")
    _i32(ctx.cu_rows, ctx.n_seqs + 1, "first rows")
    _i32(ctx.slots, ctx.n_seqs, "slots")
    y = torch.empty((n, channels), dtype=out_dtype, device=x.device)
    esize = x.element_size()
    src = x.data_ptr() + first * esize
    keep = 1 if n == ctx.n_seqs else 0
    lib = library.core()
    check(lib.sb_time_conv(_p(y), _dt(y), channels, src, _dt(x), x.shape[1], _p(weight), _dt(weight), _p(bias),
                           _dt(bias) if bias is not None else 0, _p(state), _p(ctx.row_seq), _p(ctx.cu_rows), _p(ctx.slots),
                           n, ctx.n_seqs, channels, taps, 1 if activation == "silu" else 0, 1 if residual else 0, keep, _stream()))
    if not keep:
        check(lib.sb_time_conv_keep(src, _dt(x), x.shape[1], _p(state), _p(ctx.cu_rows), _p(ctx.slots), n, ctx.n_seqs,
                                    channels, taps, _stream()))
    return y


def _f32_vec(t: torch.Tensor, n: int, what: str) -> None:
    if t.dtype != torch.float32 or t.numel() != n or not t.is_cuda or not t.is_contiguous():
        raise KernelLibraryError(f"{what} must be {n} float32 numbers on the GPU")


def _f32_rows(t: torch.Tensor, n: int, width: int, what: str) -> None:
    """``t`` float32 [n, >= width] whose rows are contiguous (a column range of wider rows is fine)."""
    if t.dtype != torch.float32 or t.dim() != 2 or t.shape[0] != n or t.shape[1] < width or t.stride(1) != 1 or not t.is_cuda:
        raise KernelLibraryError(f"{what} must be float32 rows [{n}, {width}] on the GPU, not {tuple(t.shape)}")


def state_scan_limits():
    lib = library.core()
    return int(lib.sb_state_scan_max_rows()), int(lib.sb_state_scan_max_cols())


def state_scan_chunk_rows() -> int:
    """The rows of a chunk of the chunked forms of :func:`ssd_scan` and :func:`delta_scan`."""
    return int(library.core().sb_state_scan_chunk_rows())


def _scan_chunks(chunks: Optional[torch.Tensor]) -> int:
    if chunks is None:
        return 0
    _dev(chunks)
    if chunks.dtype != torch.int32 or chunks.dim() != 2 or chunks.shape[1] != 4 or not chunks.is_contiguous() or not len(chunks):
        raise KernelLibraryError("chunks must be int32 [n, 4] with a run at least")
    return int(chunks.shape[0])


def ssd_scan(z: torch.Tensor, x: torch.Tensor, b: torch.Tensor, c: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor,
             a_log: torch.Tensor, d_skip: torch.Tensor, state: torch.Tensor, ctx, heads: int, groups: int, n_state: int,
             v_dim: int, chunks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The selective state-space recurrence over the rows of the step (see csrc/state_space.hip):
    ``z``, ``x`` [n, heads * v_dim], ``b``, ``c`` [n, groups * n_state] (column ranges of one tensor),
    ``dt`` [n, heads] before bias and softplus, all float32 (views of wider rows allowed);
    ``state`` float32 [slots, heads, n_state, v_dim], moved on.  Returns y * silu(z), float32 [n, heads * v_dim].
    ``chunks`` (int32 [m, 4], the step's rows in runs of at most :func:`state_scan_chunk_rows` rows of one
    sequence, as the context lists them): the chunked form, for long prompts."""
    n = ctx.n_rows
    inner = heads * v_dim
    _f32_rows(z, n, inner, "z")
    _f32_rows(x, n, inner, "x")
    _f32_rows(b, n, groups * n_state, "B")
    _f32_rows(c, n, groups * n_state, "C")
    _f32_rows(dt, n, heads, "dt")
    if b.stride(0) != c.stride(0) or b.untyped_storage().data_ptr() != c.untyped_storage().data_ptr():
        raise KernelLibraryError("B and C must be column ranges of the same rows")
    for t, what in ((dt_bias, "dt_bias"), (a_log, "A_log"), (d_skip, "D")):
        _f32_vec(t, heads, what)
    if state.dtype != torch.float32 or tuple(state.shape[1:]) != (heads, n_state, v_dim) or not state.is_contiguous():
        raise KernelLibraryError(f"the state must be float32 [slots, {heads}, {n_state}, {v_dim}]")
    out = torch.empty((n, inner), dtype=torch.float32, device=z.device)
    c_off = (c.data_ptr() - b.data_ptr()) // 4
    m = _scan_chunks(chunks)
    part = torch.empty((m, heads, n_state, v_dim), dtype=torch.float32, device=z.device) if m else None
    part_decay = torch.empty((m, heads), dtype=torch.float32, device=z.device) if m else None
    check(library.core().sb_ssd_scan(_p(out), inner, _p(z), z.stride(0), _p(x), x.stride(0), _p(b), b.stride(0), c_off,
                                     _p(dt), dt.stride(0), _p(dt_bias), _p(a_log), _p(d_skip), _p(state), _p(ctx.cu_rows),
                                     _p(ctx.slots), ctx.n_seqs, heads, groups, n_state, v_dim, _p(chunks), m,
                                     state_scan_chunk_rows() if m else 0, _p(part), _p(part_decay), _stream()))
    return out


def delta_scan(qkv: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor, gate: torch.Tensor, dt_bias: torch.Tensor,
               a_log: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, ctx, heads: int, kv_heads: int, dim: int,
               v_dim: int, eps: float, eps_unit: float, out_dtype: torch.dtype,
               chunks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The delta rule with a decay per key channel over the rows of the step (see csrc/state_space.hip):
    ``qkv`` [n, 2 * kv_heads * dim + heads * v_dim] after the short convolution, ``beta`` [n, heads],
    ``decay`` [n, heads * dim], ``gate`` [n, heads * v_dim] before their activations, all float32;
    ``state`` float32 [slots, heads, dim, v_dim], moved on.  Returns the normed, gated heads
    [n, heads * v_dim] in ``out_dtype``.  ``chunks``: as for :func:`ssd_scan`."""
    n = ctx.n_rows
    _f32_rows(qkv, n, 2 * kv_heads * dim + heads * v_dim, "q, k and v")
    _f32_rows(beta, n, heads, "beta")
    _f32_rows(decay, n, heads * dim, "the decays")
    _f32_rows(gate, n, heads * v_dim, "the gate")
    _f32_vec(dt_bias, heads * dim, "dt_bias")
    _f32_vec(a_log, heads, "A_log")
    _dev(weight)
    if weight.numel() != v_dim:
        raise KernelLibraryError(f"the norm's weight has {weight.numel()} elements for values of {v_dim}")
    if state.dtype != torch.float32 or tuple(state.shape[1:]) != (heads, dim, v_dim) or not state.is_contiguous():
        raise KernelLibraryError(f"the state must be float32 [slots, {heads}, {dim}, {v_dim}]")
    out = torch.empty((n, heads * v_dim), dtype=out_dtype, device=qkv.device)
    m = _scan_chunks(chunks)
    part = torch.empty((m, heads, dim, v_dim + dim), dtype=torch.float32, device=qkv.device) if m else None
    check(library.core().sb_delta_scan(_p(out), _dt(out), heads * v_dim, _p(qkv), qkv.stride(0), _p(beta), beta.stride(0),
                                       _p(decay), decay.stride(0), _p(gate), gate.stride(0), _p(dt_bias), _p(a_log),
                                       _p(weight), _dt(weight), _p(state), _p(ctx.cu_rows), _p(ctx.slots), ctx.n_seqs, heads,
                                       kv_heads, dim, v_dim, float(eps), float(eps_unit), _p(chunks), m,
                                       state_scan_chunk_rows() if m else 0, _p(part), _stream()))
    return out


def qk_rownorm_store(qk: torch.Tensor, q_dtype: torch.dtype, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                     eps: float, temp_coef: float, temp_every: int, row_pos: torch.Tensor, row_seq: torch.Tensor,
                     k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], page_table: Optional[torch.Tensor],
                     heads_q: int, heads_kv: int, head_dim: int, store: bool = True, values_from_keys: bool = True) -> torch.Tensor:
    """Queries and keys normed over their whole projections (see csrc/attention_mixed.hip): from float32
    rows [q | k] the queries in ``q_dtype``, times the temperature of the row's position; with ``store``
    the normed keys into the key cache and, with ``values_from_keys``, the keys as they came into the
    value cache."""
    _dev(qk, q_weight, k_weight, row_pos, row_seq, k_cache, v_cache, page_table)
    n = qk.shape[0]
    qw, kw = heads_q * head_dim, heads_kv * head_dim
    if qk.dtype != torch.float32 or qk.dim() != 2 or qk.shape[1] < qw + (kw if store else 0):
        raise KernelLibraryError(f"the projections must be float32 [rows, {qw + (kw if store else 0)}]")
    for w, m, what in ((q_weight, qw, "query"), (k_weight, kw, "key")):
        if w is not None and (w.numel() != m or (q_weight is not None and w.dtype != q_weight.dtype)):
            raise KernelLibraryError(f"the {what} norm's weight must have {m} elements (and both one type)")
    _i32(row_pos, n, "row positions")
    max_pages = n_pages = cache_dt = 0
    if store:
        _check_cache_kv(k_cache, v_cache, heads_kv, head_dim, head_dim)
        _check_rows(row_pos, row_seq, page_table, n)
        max_pages, n_pages, cache_dt = page_table.shape[1], k_cache.shape[0], _dt(k_cache)
    q = torch.empty((n, qw), dtype=q_dtype, device=qk.device)
    wt = q_weight if q_weight is not None else k_weight
    check(library.core().sb_qk_rownorm_store(
        _p(q), _dt(q), _p(qk), qk.shape[1], _p(q_weight), _p(k_weight), _dt(wt) if wt is not None else 0, float(eps),
        float(temp_coef), int(temp_every), _p(row_pos), _p(row_seq), _p(page_table) if store else None, max_pages, n_pages,
        _p(k_cache) if store else None, _p(v_cache) if store else None, cache_dt, n, heads_q, heads_kv, head_dim,
        1 if store else 0, 1 if values_from_keys else 0, _stream()))
    return q


def attention_shared_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                           row_pos: torch.Tensor, row_seq: torch.Tensor, heads_q: int, heads_kv: int, head_dim: int,
                           v_dim: int, scale: float, r1: Optional[torch.Tensor], r2: Optional[torch.Tensor]) -> torch.Tensor:
    """O[row, g, c] = sum_j P_g(row, j) V_c(j): every query head's causal softmax (scores times ``scale``
    minus r1_g ln(1 + r2_g distance)) applied to the values of every key/value head; float32
    [rows, heads_q, heads_kv, v_dim].  One wave per (row, g, c)."""
    _dev(q, k_cache, v_cache, page_table, row_pos, row_seq, r1, r2)
    n = q.shape[0]
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim:
        raise KernelLibraryError(f"queries must be [rows, {heads_q * head_dim}]")
    _check_cache_kv(k_cache, v_cache, heads_kv, head_dim, v_dim)
    _check_rows(row_pos, row_seq, page_table, n)
    if (r1 is None) != (r2 is None):
        raise KernelLibraryError("the distance bias needs both of its numbers a head")
    if r1 is not None:
        _f32_vec(r1, heads_q, "r1")
        _f32_vec(r2, heads_q, "r2")
    out = torch.empty((n, heads_q, heads_kv, v_dim), dtype=torch.float32, device=q.device)
    check(library.core().sb_attention_shared(_p(out), _p(q), _dt(q), _p(k_cache), _p(v_cache), _dt(k_cache), _p(page_table),
                                             page_table.shape[1], k_cache.shape[0], _p(row_pos), _p(row_seq), n, heads_q,
                                             heads_kv, head_dim, v_dim, float(scale), _p(r1), _p(r2), _stream()))
    return out


def head_mix(o: torch.Tensor, mix: Optional[torch.Tensor], out_dtype: torch.dtype) -> torch.Tensor:
    """out[row, h] = sum_g mix[h, g] o[row, g, kv(h)] for ``o`` [rows, heads_q, heads_kv, v_dim], float32 or
    bfloat16 (``mix`` None: the identity); [rows, heads_q * v_dim] in ``out_dtype``."""
    _dev(o, mix)
    if o.dim() != 4:
        raise KernelLibraryError("the heads' results must be [rows, heads_q, heads_kv, v_dim]")
    n, hq, hkv, vd = o.shape
    if mix is not None and tuple(mix.shape) != (hq, hq):
        raise KernelLibraryError(f"the heads' mixing matrix must be [{hq}, {hq}]")
    out = torch.empty((n, hq * vd), dtype=out_dtype, device=o.device)
    check(library.core().sb_head_mix(_p(out), _dt(out), _p(o), _dt(o), _p(mix), _dt(mix) if mix is not None else 0, n, hq, hkv,
                                     vd, _stream()))
    return out


def shared_attention_mfma_ok(q_dtype, cache_dtype, head_dim: int, v_dim: int) -> bool:
    return capped_attention_mfma_ok(q_dtype, cache_dtype, head_dim, v_dim)


def attention_shared_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                          row_pos: torch.Tensor, tiles: torch.Tensor, heads_q: int, heads_kv: int, head_dim: int, v_dim: int,
                          scale: float, r1: Optional[torch.Tensor], r2: Optional[torch.Tensor],
                          chunks: Optional[int] = None) -> torch.Tensor:
    """The matrix-core form of :func:`attention_shared_plain` (the kernels of :func:`attention_capped_mfma`
    with the distance bias and every kv head's values): bfloat16 [rows, heads_q, heads_kv, v_dim].
    ``tiles`` int32 [n, 4]: the rows in runs of up to 16 consecutive rows of one sequence."""
    _dev(q, k_cache, v_cache, page_table, row_pos, tiles, r1, r2)
    n = q.shape[0]
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim or q.dtype != torch.bfloat16:
        raise KernelLibraryError(f"queries must be bfloat16 [rows, {heads_q * head_dim}]")
    _check_cache_kv(k_cache, v_cache, heads_kv, head_dim, v_dim)
    if k_cache.dtype != torch.bfloat16:
        raise KernelLibraryError("the matrix-core kernel reads a bfloat16 cache")
    _i32(row_pos, n, "row positions")
    if page_table.dtype != torch.int32 or page_table.dim() != 2:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")
    if tiles.dtype != torch.int32 or tiles.dim() != 2 or tiles.shape[1] != 4:
        raise KernelLibraryError("row tiles must be int32 [n, 4]")
    if (r1 is None) != (r2 is None):
        raise KernelLibraryError("the distance bias needs both of its numbers a head")
    if r1 is not None:
        _f32_vec(r1, heads_q, "r1")
        _f32_vec(r2, heads_q, "r2")
    n_tiles, max_pages = tiles.shape[0], page_table.shape[1]
    group = heads_q // heads_kv
    blocks = max(1, n_tiles * heads_kv * heads_kv * ((group + 3) // 4))
    if chunks is None:
        chunks = max(1, min(max_pages, CAPPED_SPLIT_BLOCKS // blocks))
    chunk_pages = (max_pages + chunks - 1) // chunks
    chunks = (max_pages + chunk_pages - 1) // chunk_pages
    part_o = part_ml = None
    if chunks > 1:
        part_o = torch.empty((chunks, n, heads_q * heads_kv, v_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((chunks, n, heads_q * heads_kv, 2), dtype=torch.float32, device=q.device)
    out = torch.empty((n, heads_q, heads_kv, v_dim), dtype=torch.bfloat16, device=q.device)
    lib = library.capped_attention_library(head_dim, v_dim)
    check(lib.sb_cattn_shared_bf16(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(page_table), max_pages, k_cache.shape[0],
                                   _p(row_pos), _p(tiles), n_tiles, n, heads_q, heads_kv, float(scale), 0, 0.0, 0, chunks,
                                   chunk_pages, _p(part_o), _p(part_ml), _p(r1), _p(r2), 1, _stream()),
          lib, "sb_cattn_last_error")
    return out


def attention_shared(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor, ctx,
                     heads_q: int, heads_kv: int, head_dim: int, v_dim: int, scale: float, r1: Optional[torch.Tensor],
                     r2: Optional[torch.Tensor], mix: Optional[torch.Tensor], out_dtype: torch.dtype,
                     fast: bool = True) -> torch.Tensor:
    """Attention of a step's rows over the cache with a distance bias and the heads' weights mixed by
    ``mix`` [heads_q, heads_q]: every query head's weights against every key/value head's values, then the
    mix of the results; [rows, heads_q * v_dim] in ``out_dtype``.  bfloat16 with head sizes in steps of 16
    runs on the matrix cores; everything else takes the plain kernel."""
    if fast and shared_attention_mfma_ok(q.dtype, k_cache.dtype, head_dim, v_dim):
        o = attention_shared_mfma(q, k_cache, v_cache, page_table, ctx.row_pos, ctx.row_tiles(CAPPED_ROW_TILE), heads_q,
                                  heads_kv, head_dim, v_dim, scale, r1, r2)
    else:
        o = attention_shared_plain(q, k_cache, v_cache, page_table, ctx.row_pos, ctx.row_seq, heads_q, heads_kv, head_dim,
                                   v_dim, scale, r1, r2)
    return head_mix(o, mix, out_dtype)

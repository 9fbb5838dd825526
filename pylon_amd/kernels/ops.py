"""Tensor-level wrappers of the HIP entry points.

Every wrapper checks device, element type, contiguity and shapes on the host before
it launches, and launches on torch's current stream.  None has a CPU path.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import library as _lib
from . import plan
from .library import KernelError

F32 = 0
BF16 = 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


def compute_units() -> int:
    """Compute units of the current device."""
    return _lib.compute_units()


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"the kernels take float32 and bfloat16, not {dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    """The current stream's handle.  A step asks for it once per launch, a few hundred times:
    the two raw calls take a fifth of a microsecond, ``torch.cuda.current_stream()`` six."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(t: Optional[torch.Tensor], name: str, dtype=None) -> int:
    """Device pointer of a checked tensor (0 for None)."""
    if t is None:
        return 0
    if not t.is_cuda:
        raise KernelError(f"{name} must live on the GPU; there is no CPU path")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    return t.data_ptr()


def embed(ids: torch.Tensor, table: torch.Tensor, *, scale: float = 1.0,
          out: Optional[torch.Tensor] = None, chosen: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 ``out[t] = table[ids[t]] * scale``.  With ``chosen`` (int32, on the device) an
    id ``-(1 + s)`` is replaced by ``chosen[s]``: the token a sampler left there."""
    tokens = ids.numel()
    vocab, hidden = table.shape
    if out is None:
        out = torch.empty((tokens, hidden), dtype=torch.float32, device=table.device)
    elif out.shape != (tokens, hidden):
        raise KernelError(f"embed: out has shape {tuple(out.shape)}, expected {(tokens, hidden)}")
    _lib.call("pylon_embed", _dev(out, "out", torch.float32), _dev(table, "table"),
              dtype_code(table.dtype), _dev(ids, "ids", torch.int32),
              None if chosen is None else _dev(chosen, "chosen", torch.int32), tokens, hidden, vocab,
              float(scale), _stream())
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, *, out_dtype=None,
            row_idx: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``(x / sqrt(mean(x^2) + eps)) * weight`` over the last axis of a 2-D tensor."""
    if x.dim() != 2:
        raise KernelError("rmsnorm takes a 2-D input")
    dim = x.shape[1]
    if weight.shape != (dim,):
        raise KernelError(f"rmsnorm: weight has shape {tuple(weight.shape)}, expected ({dim},)")
    rows = x.shape[0] if row_idx is None else row_idx.numel()
    out_dtype = out_dtype or x.dtype
    if out is None:
        out = torch.empty((rows, dim), dtype=out_dtype, device=x.device)
    elif out.shape != (rows, dim):
        raise KernelError("rmsnorm: out has the wrong shape")
    _lib.call("pylon_rmsnorm", _dev(out, "out"), dtype_code(out.dtype), _dev(x, "x"),
              dtype_code(x.dtype), _dev(weight, "weight", torch.float32),
              _dev(row_idx, "row_idx", torch.int32), rows, dim, float(eps), _stream())
    return out


def add_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, *, row_idx: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``resid += delta`` (float32, in place) and the RMSNorm of the sum.

    ``delta`` has the residual's shape, or is a stack ``[parts, tokens, dim]`` of partial
    sums that are added up first.  With ``row_idx`` only those rows are normed and
    ``resid`` is left as it is.
    """
    if resid.dim() != 2:
        raise KernelError("add_rmsnorm takes a 2-D residual")
    dim = resid.shape[1]
    n_delta, delta_stride = 1, 0
    if delta is not None:
        if delta.dim() == 3:
            n_delta, delta_stride = delta.shape[0], delta.shape[1] * delta.shape[2]
            if delta.shape[1:] != resid.shape:
                raise KernelError("add_rmsnorm: partial sums and resid differ in shape")
        elif delta.shape != resid.shape:
            raise KernelError("add_rmsnorm: delta and resid differ in shape")
    if weight.shape != (dim,):
        raise KernelError(f"add_rmsnorm: weight has shape {tuple(weight.shape)}, expected ({dim},)")
    rows = resid.shape[0] if row_idx is None else row_idx.numel()
    if out is None:
        out = torch.empty((rows, dim), dtype=out_dtype, device=resid.device)
    elif out.shape != (rows, dim) or out.dtype != out_dtype:
        raise KernelError("add_rmsnorm: out has the wrong shape or dtype")
    _lib.call("pylon_add_rmsnorm", _dev(out, "out"), dtype_code(out.dtype),
              _dev(resid, "resid", torch.float32), _dev(delta, "delta"),
              dtype_code(delta.dtype) if delta is not None else F32, n_delta, delta_stride,
              _dev(weight, "weight", torch.float32), _dev(row_idx, "row_idx", torch.int32),
              rows, dim, float(eps), _stream())
    return out


def residual_add(resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    if delta.shape != resid.shape:
        raise KernelError("residual_add: shapes differ")
    _lib.call("pylon_residual_add", _dev(resid, "resid", torch.float32), _dev(delta, "delta"),
              dtype_code(delta.dtype), resid.numel(), _stream())
    return resid


def silu_gate(gate_up: torch.Tensor, *, out_dtype: Optional[torch.dtype] = None,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate_up[:, :I]) * gate_up[:, I:]`` for a ``[tokens, 2I]`` input; the result may
    have another element type than the input (float32 sums in, bfloat16 out: one rounding)."""
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise KernelError("silu_gate takes a [tokens, 2*I] input")
    tokens, two_i = gate_up.shape
    inter = two_i // 2
    out_dtype = out_dtype or (out.dtype if out is not None else gate_up.dtype)
    if out is None:
        out = torch.empty((tokens, inter), dtype=out_dtype, device=gate_up.device)
    elif out.shape != (tokens, inter) or out.dtype != out_dtype:
        raise KernelError("silu_gate: out has the wrong shape or dtype")
    _lib.call("pylon_silu_gate", _dev(out, "out"), dtype_code(out.dtype), _dev(gate_up, "gate_up"),
              dtype_code(gate_up.dtype), tokens, inter, _stream())
    return out


def qkv_prepare(qkv: torch.Tensor, q_out: torch.Tensor, k_cache: Optional[torch.Tensor],
                v_cache: Optional[torch.Tensor], *, n_heads: int, n_kv_heads: int, head_dim: int,
                q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                inv_freq: Optional[torch.Tensor], rot_dim: int, positions: Optional[torch.Tensor],
                slot_map: Optional[torch.Tensor], store_kv: bool) -> None:
    """Per-head norm and rotation of q and k; q to ``q_out``; k and v into cache slots."""
    if qkv.dim() != 2:
        raise KernelError("qkv_prepare takes a 2-D projection output")
    tokens, width = qkv.shape
    heads = n_heads + (2 * n_kv_heads if store_kv else 0)
    if width != heads * head_dim:
        raise KernelError(f"qkv_prepare: projection width {width} is not {heads} heads of {head_dim}")
    if q_out.shape != (tokens, n_heads, head_dim) or q_out.dtype != qkv.dtype:
        raise KernelError("qkv_prepare: q_out has the wrong shape or dtype")
    for name, wt in (("q_weight", q_weight), ("k_weight", k_weight)):
        if wt is not None and wt.shape != (head_dim,):
            raise KernelError(f"qkv_prepare: {name} must have shape ({head_dim},)")
    if inv_freq is not None and inv_freq.numel() != rot_dim // 2:
        raise KernelError("qkv_prepare: inv_freq must hold rot_dim/2 frequencies")
    if positions is not None and positions.numel() != tokens:
        raise KernelError("qkv_prepare: one position per token is required")
    if store_kv:
        if k_cache is None or v_cache is None or slot_map is None:
            raise KernelError("qkv_prepare: storing needs k_cache, v_cache and slot_map")
        if slot_map.numel() != tokens:
            raise KernelError("qkv_prepare: one cache slot per token is required")
        for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c.dtype != qkv.dtype or c.shape[-2:] != (n_kv_heads, head_dim):
                raise KernelError(f"qkv_prepare: {name} must be [..., {n_kv_heads}, {head_dim}] of {qkv.dtype}")
    _lib.call("pylon_qkv_prepare", _dev(q_out, "q_out"), _dev(k_cache if store_kv else None, "k_cache"),
              _dev(v_cache if store_kv else None, "v_cache"), _dev(qkv, "qkv"), dtype_code(qkv.dtype),
              width, _dev(q_weight, "q_weight", torch.float32), _dev(k_weight, "k_weight", torch.float32),
              float(eps), _dev(inv_freq, "inv_freq", torch.float32), int(rot_dim),
              _dev(positions, "positions", torch.int32), _dev(slot_map if store_kv else None, "slot_map", torch.int32),
              tokens, n_heads, n_kv_heads, head_dim, 1 if store_kv else 0, _stream())


def mask_code(window: Optional[int], chunk: Optional[int] = None) -> int:
    """The one integer by which the attention kernels are told which earlier keys a token sees:
    ``w > 0`` the last ``w`` (itself included), ``-c < 0`` those of its own chunk of ``c``
    positions (chunks counted from the request's first token), 0 all of them."""
    if window is not None and chunk is not None:
        raise KernelError("a mask is a window or chunks, not both")
    if window is not None:
        if window < 1:
            raise KernelError("a window holds at least one key")
        return int(window)
    if chunk is not None:
        if chunk < 1:
            raise KernelError("a chunk holds at least one position")
        return -int(chunk)
    return 0


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, tok_row: torch.Tensor, positions: torch.Tensor, *,
                    page_size: int, window: Optional[int], scale: float,
                    out: Optional[torch.Tensor] = None, rel: Optional[torch.Tensor] = None,
                    bucket: Optional[torch.Tensor] = None, sink: bool = False,
                    v_transposed: bool = False, chunk: Optional[int] = None,
                    log_bias: Optional[torch.Tensor] = None, softcap: Optional[float] = None,
                    sink_logit: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of each token over its request's cached keys ``<=`` its position (with
    ``window`` the last so many, with ``chunk`` those of its own chunk: :func:`mask_code`).
    ``q`` is ``[tokens, heads, head_dim]`` and may be a slice of wider rows (a fused
    projection); values may have another size than keys.  ``rel`` (float32 ``[rows, heads]``)
    with ``bucket`` (int32 ``[n]``) adds ``rel[bucket[min(i - j, n - 1)], head]`` to the scaled
    score of query ``i`` and key ``j``; ``log_bias`` (float32 ``[2, heads]``: ``a`` then ``b``) takes
    ``a[head] * log(1 + b[head] * (i - j))`` off it instead; ``sink`` adds one to the softmax's
    denominator.  With ``v_transposed`` the values lie as ``[pages, kv_heads, v_dim, page_size]``.
    ``softcap``: the scaled score ``s`` becomes ``softcap * tanh(s / softcap)``.  ``sink_logit``
    (float32 ``[heads]``): ``exp(sink_logit[head])`` joins the denominator, unscaled and uncapped."""
    if q.dim() != 3:
        raise KernelError("paged_attention takes q as [tokens, heads, head_dim]")
    if sink_logit is not None and (sink or sink_logit.shape != (q.shape[1],)):
        raise KernelError("paged_attention: sink_logit is float32 [heads], and not together with the fixed sink")
    if softcap is not None and not softcap > 0:
        raise KernelError("paged_attention: a soft cap is positive")
    tokens, n_heads, head_dim = q.shape
    if v_transposed and v_cache.dim() == 4:
        v_shape = (v_cache.shape[0], v_cache.shape[3], v_cache.shape[1], v_cache.shape[2])
    else:
        v_shape = tuple(v_cache.shape)
    if k_cache.dim() != 4 or v_cache.dim() != 4 or tuple(k_cache.shape[:3]) != v_shape[:3]:
        raise KernelError("paged_attention: caches must be [pages, page_size, kv_heads, head_dim]")
    pages, psize, n_kv_heads, hd = k_cache.shape
    v_dim = v_shape[3]
    if q.stride(2) != 1 or q.stride(1) != head_dim or (tokens > 1 and q.stride(0) < n_heads * head_dim):
        raise KernelError("paged_attention: the heads of a q row must lie side by side")
    if (rel is None) != (bucket is None):
        raise KernelError("paged_attention: rel and bucket go together")
    if rel is not None and (rel.dim() != 2 or rel.shape[1] != n_heads or bucket.numel() < 1):
        raise KernelError("paged_attention: rel must be [rows, heads] and bucket hold at least one entry")
    if log_bias is not None:
        if rel is not None or log_bias.shape != (2, n_heads) or not log_bias.is_contiguous():
            raise KernelError("paged_attention: log_bias is float32 [2, heads], and not together with a table")
        rel = log_bias
    if psize != page_size or hd != head_dim:
        raise KernelError("paged_attention: cache geometry does not match page_size/head_dim")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError("paged_attention: q and the caches differ in dtype")
    if pages * page_size >= 2 ** 31:
        raise KernelError("paged_attention: the cache holds more slots than an int32 can index")
    if block_table.dim() != 2:
        raise KernelError("paged_attention: block_table must be [rows, width]")
    if tok_row.numel() != tokens or positions.numel() != tokens:
        raise KernelError("paged_attention: one row id and one position per token are required")
    if out is None:
        out = torch.empty((tokens, n_heads, v_dim), dtype=q.dtype, device=q.device)
    elif out.shape != (tokens, n_heads, v_dim) or out.dtype != q.dtype:
        raise KernelError("paged_attention: out has the wrong shape or dtype")
    if not q.is_cuda:
        raise KernelError("q must live on the GPU; there is no CPU path")
    _lib.call("pylon_paged_attention", _dev(out, "out"), q.data_ptr(), _dev(k_cache, "k_cache"),
              _dev(v_cache, "v_cache"), dtype_code(q.dtype), _dev(block_table, "block_table", torch.int32),
              block_table.shape[1], _dev(tok_row, "tok_row", torch.int32),
              _dev(positions, "positions", torch.int32), tokens, n_heads, n_kv_heads, head_dim,
              page_size, mask_code(window, chunk), float(scale), v_dim, q.stride(0) if tokens > 1 else n_heads * head_dim,
              _dev(rel, "rel", torch.float32), _dev(bucket, "bucket", torch.int32),
              0 if bucket is None else bucket.numel(), 1 if sink else 0, 1 if v_transposed else 0,
              float(softcap or 0.0), _dev(sink_logit, "sink_logit", torch.float32), _stream())
    return out


SINK_MAX_BIAS = 4096  # distances the matrix-core sink attention keeps a bias for in LDS
SINK_TILE = 32        # most tokens of one tile of it


def attention_sink_ok(dtype: torch.dtype, *, head_dim: int, v_dim: int, page_size: int, bucket_len: int) -> bool:
    """Whether the matrix-core kernel takes this geometry (else the general kernel does)."""
    return (dtype == torch.bfloat16 and head_dim % 8 == 0 and 8 <= head_dim <= 256 and v_dim % 4 == 0
            and 4 <= v_dim <= 256 and page_size % 32 == 0 and bucket_len <= SINK_MAX_BIAS)


def sink_cuts(tokens: int, n_heads: int, n_kv_heads: int, max_len: int, units: Optional[int] = None) -> int:
    """Workgroups that share the keys of one (token, key/value head) in a step of single tokens:
    more than one while the launch would leave compute units idle and every cut keeps at least
    256 keys of the longest request (``max_len`` may be an upper bound)."""
    units = units or _lib.compute_units()
    group = n_heads // n_kv_heads
    groups = tokens * n_kv_heads * (-(-group // 4))
    cuts = 1
    while cuts < 64 and groups * cuts * 2 <= 2 * units and max_len >= cuts * 2 * 256:
        cuts *= 2
    return cuts


def bias_by_distance(rel: torch.Tensor, bucket: torch.Tensor) -> torch.Tensor:
    """float32 ``[heads, n]``: ``rel[bucket[d], head]`` for every distance ``d`` the bucket table
    lists: a learned bias table looked up once, for kernels that keep a head's biases in LDS."""
    return rel.float().index_select(0, bucket.long()).t().contiguous()


def attention_sink(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                   tiles: Optional[torch.Tensor], positions: Optional[torch.Tensor], *, page_size: int, scale: float,
                   bias: Optional[torch.Tensor], sink: bool, cuts: int = 1, window: Optional[int] = None,
                   chunk: Optional[int] = None, softcap: Optional[float] = None,
                   sink_logit: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention with a bias by distance and a sink on the matrix cores: bfloat16 ``q``
    ``[tokens, heads, head_dim]`` (maybe a slice of wider rows), keys ``[pages, page_size, kv_heads,
    head_dim]``, values transposed inside their pages ``[pages, kv_heads, v_dim, page_size]``.
    ``bias`` float32 ``[heads, n]``: what is added to the scaled score at distance ``min(i - j, n - 1)``.
    ``tiles`` int32 ``[n, 4]`` (first token, count <= 32, block-table row, first position); or None
    with ``positions``: every token a tile of its own on its own row of the table.  ``cuts``
    workgroups share the keys of a tile and a second kernel merges their float partial results.
    ``window`` / ``chunk``: which earlier keys a token sees (:func:`mask_code`).  ``softcap``: the
    scaled score ``s`` becomes ``softcap * tanh(s / softcap)`` before the bias; ``sink_logit`` (float32
    ``[heads]``, with ``sink``): the sink's score per head in place of 0."""
    if q.dim() != 3 or k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelError("attention_sink takes q [tokens, heads, head_dim] and 4-D caches")
    if sink_logit is not None and (not sink or sink_logit.shape != (q.shape[1],)):
        raise KernelError("attention_sink: sink_logit is float32 [heads] and goes with sink")
    if softcap is not None and not softcap > 0:
        raise KernelError("attention_sink: a soft cap is positive")
    tokens, n_heads, head_dim = q.shape
    pages, psize, n_kv_heads, hd = k_cache.shape
    v_dim = v_cache.shape[2]
    if v_cache.shape != (pages, n_kv_heads, v_dim, psize) or psize != page_size or hd != head_dim:
        raise KernelError("attention_sink: cache geometry does not match page_size/head_dim")
    if not attention_sink_ok(q.dtype, head_dim=head_dim, v_dim=v_dim, page_size=page_size,
                             bucket_len=0 if bias is None else bias.shape[-1]):
        raise KernelError("attention_sink does not take this geometry")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype or n_heads % n_kv_heads:
        raise KernelError("attention_sink: q and the caches differ in dtype, or the heads do not group")
    if q.stride(2) != 1 or q.stride(1) != head_dim or (tokens > 1 and q.stride(0) < n_heads * head_dim):
        raise KernelError("attention_sink: the heads of a q row must lie side by side")
    if pages * page_size >= 2 ** 31 or block_table.dim() != 2:
        raise KernelError("attention_sink: the cache is too large for int32 slots, or the table is not 2-D")
    if bias is not None and (bias.dim() != 2 or bias.shape[0] != n_heads):
        raise KernelError("attention_sink: bias must be [heads, distances]")
    if tiles is not None:
        if tiles.dim() != 2 or tiles.shape[1] != 4:
            raise KernelError("attention_sink: tiles must be [n, 4]")
        n_tiles = tiles.shape[0]
    else:
        if positions is None or positions.numel() != tokens or block_table.shape[0] < tokens:
            raise KernelError("attention_sink: without tiles, one position and one table row per token")
        n_tiles = tokens
    out = torch.empty((tokens, n_heads, v_dim), dtype=q.dtype, device=q.device)
    partial = None
    if cuts > 1:
        partial = torch.empty((tokens * n_heads * cuts * (2 + v_dim),), dtype=torch.float32, device=q.device)
    _lib.call("pylon_attention_sink", _dev(out, "out"), q.data_ptr(), q.stride(0) if tokens > 1 else n_heads * head_dim,
              _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"), _dev(block_table, "block_table", torch.int32),
              block_table.shape[1], _dev(tiles, "tiles", torch.int32), _dev(positions, "positions", torch.int32),
              n_tiles, n_heads, n_kv_heads, head_dim, v_dim, page_size, float(scale), _dev(bias, "bias", torch.float32),
              0 if bias is None else bias.shape[1], 1 if sink else 0, int(cuts), _dev(partial, "partial"),
              0 if partial is None else partial.numel(), tokens, mask_code(window, chunk), float(softcap or 0.0),
              _dev(sink_logit, "sink_logit", torch.float32), _stream())
    return out


def add_normed_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], gain: Optional[torch.Tensor], eps: float,
                       out_dtype: Optional[torch.dtype], *, post_gain: Optional[torch.Tensor] = None,
                       post_eps: float = 0.0, row_idx: Optional[torch.Tensor] = None,
                       delta_scale: Optional[torch.Tensor] = None,
                       delta_bias: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``resid += post_gain * d / rms(d)`` (``d`` = ``delta``, or the sum of a stack of float32
    partial sums; without ``post_gain``: ``resid += d``), in float32 and in place, then
    ``gain * resid / rms(resid)`` in ``out_dtype``, with ``rms(v) = sqrt(mean(v^2) + eps)``.
    ``post_gain`` is one float32 number on the device; ``gain`` one number or one per element.
    With ``row_idx`` only those rows are normed and ``resid`` is left as it is; with
    ``gain`` None only the sum is formed.  ``delta_bias`` (float32 ``[dim]``) is added to ``d``
    first; with ``delta_scale`` (float32 ``[dim]``, not together with ``post_gain``) the sum is
    ``resid += delta_scale * d``."""
    if resid.dim() != 2:
        raise KernelError("add_normed_rmsnorm takes a 2-D residual")
    dim = resid.shape[1]
    for name, vector in (("delta_scale", delta_scale), ("delta_bias", delta_bias)):
        if vector is not None and (vector.shape != (dim,) or delta is None):
            raise KernelError(f"add_normed_rmsnorm: {name} is one number per element of an output that is given")
    n_delta, delta_stride = 1, 0
    if delta is not None:
        if delta.dim() == 3:
            n_delta, delta_stride = delta.shape[0], delta.shape[1] * delta.shape[2]
            if delta.shape[1:] != resid.shape:
                raise KernelError("add_normed_rmsnorm: partial sums and resid differ in shape")
        elif delta.shape != resid.shape:
            raise KernelError("add_normed_rmsnorm: delta and resid differ in shape")
    if post_gain is not None and post_gain.numel() != 1:
        raise KernelError("add_normed_rmsnorm: post_gain is one number")
    gain_stride = 0
    if gain is not None:
        if gain.numel() == dim and gain.dim() == 1 and dim > 1:
            gain_stride = 1
        elif gain.numel() != 1:
            raise KernelError(f"add_normed_rmsnorm: gain must be one number or ({dim},)")
    rows = resid.shape[0] if row_idx is None else row_idx.numel()
    out = None
    if gain is not None:
        out = torch.empty((rows, dim), dtype=out_dtype, device=resid.device)
    _lib.call("pylon_add_normed_rmsnorm", _dev(out, "out"), dtype_code(out.dtype) if out is not None else F32,
              _dev(resid, "resid", torch.float32), _dev(delta, "delta"),
              dtype_code(delta.dtype) if delta is not None else F32, n_delta, delta_stride,
              _dev(post_gain, "post_gain", torch.float32), float(post_eps), _dev(gain, "gain", torch.float32),
              gain_stride, _dev(row_idx, "row_idx", torch.int32), rows, dim, float(eps),
              _dev(delta_scale, "delta_scale", torch.float32), _dev(delta_bias, "delta_bias", torch.float32), _stream())
    return out


def depth_mix(resid: torch.Tensor, delta: Optional[torch.Tensor], streams: torch.Tensor, index: int,
              coeff: torch.Tensor, *, delta_scale: Optional[torch.Tensor] = None,
              delta_bias: Optional[torch.Tensor] = None, gain: Optional[torch.Tensor] = None, eps: float = 0.0,
              out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """A layer's result joins the earlier layers' and the stream becomes their learned mix:
    ``X = resid + delta_scale * (d + delta_bias)`` (``d`` = ``delta`` or the sum of a stack of partial
    sums; scale and bias optional), ``streams[index] = X``, ``resid = sum_{j <= index} coeff[j] *
    streams[j]``, all float32 and in place; with ``gain`` (float32 ``[dim]``) also the norm
    ``gain * resid / sqrt(mean(resid^2) + eps)`` in ``out_dtype``.  ``streams`` is float32
    ``[n, tokens, dim]`` with ``n > index``; ``coeff`` float32 with at least ``index + 1`` numbers."""
    if resid.dim() != 2 or resid.dtype != torch.float32 or not resid.is_contiguous():
        raise KernelError("depth_mix takes a contiguous float32 2-D residual")
    rows, dim = resid.shape
    if (streams.dim() != 3 or streams.dtype != torch.float32 or streams.shape[1:] != resid.shape
            or not streams.is_contiguous() or not 0 <= index < streams.shape[0]):
        raise KernelError("depth_mix: streams must be float32 [more than index, tokens, dim]")
    if coeff.dim() != 1 or coeff.numel() < index + 1:
        raise KernelError(f"depth_mix: stream {index} needs {index + 1} coefficients")
    n_delta, delta_stride = 1, 0
    if delta is not None:
        if delta.dim() == 3:
            n_delta, delta_stride = delta.shape[0], delta.shape[1] * delta.shape[2]
            if delta.shape[1:] != resid.shape:
                raise KernelError("depth_mix: partial sums and resid differ in shape")
        elif delta.shape != resid.shape:
            raise KernelError("depth_mix: delta and resid differ in shape")
    for name, vector in (("delta_scale", delta_scale), ("delta_bias", delta_bias), ("gain", gain)):
        if vector is not None and vector.shape != (dim,):
            raise KernelError(f"depth_mix: {name} is one number per element")
    out = None if gain is None else torch.empty((rows, dim), dtype=out_dtype, device=resid.device)
    _lib.call("pylon_depth_mix", _dev(out, "out"), dtype_code(out.dtype) if out is not None else F32,
              _dev(resid, "resid", torch.float32), _dev(delta, "delta"),
              dtype_code(delta.dtype) if delta is not None else F32, n_delta, delta_stride,
              _dev(delta_scale, "delta_scale", torch.float32), _dev(delta_bias, "delta_bias", torch.float32),
              _dev(streams, "streams", torch.float32), rows * dim, int(index), _dev(coeff, "coeff", torch.float32),
              _dev(gain, "gain", torch.float32), rows, dim, float(eps), _stream())
    return out


def token_shift(h: torch.Tensor, shift: torch.Tensor, state: torch.Tensor, row_start: torch.Tensor,
                row_slots: torch.Tensor, *, rows: int, max_count: int, out_dtype: torch.dtype) -> torch.Tensor:
    """``h[t] + (h[t - 1] - h[t]) * shift`` per channel and request, zeros before a request's first
    token.  ``state`` (float32 ``[slots, width]``) holds every request's last input and is brought
    up to date; ``max_count`` bounds the tokens of a row."""
    if h.dim() != 2 or shift.shape != (h.shape[1],) or not h.is_contiguous():
        raise KernelError("token_shift takes h [tokens, width] and one weight per channel")
    tokens, width = h.shape
    if state is None or state.dim() != 2 or state.shape[1] != width:
        raise KernelError(f"token_shift: state must be [slots, {width}]")
    if row_start.numel() != rows + 1 or row_slots.numel() != rows:
        raise KernelError("token_shift: one start per row and one more, and one slot per row")
    out = torch.empty((tokens, width), dtype=out_dtype, device=h.device)
    _lib.call("pylon_token_shift", _dev(out, "out"), dtype_code(out_dtype), _dev(h, "h"), dtype_code(h.dtype),
              _dev(shift, "shift", torch.float32), _dev(state, "state", torch.float32),
              _dev(row_start, "row_start", torch.int32), _dev(row_slots, "row_slots", torch.int32), rows,
              int(max_count), width, _stream())
    return out


def add_sinusoid(x: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """``x[t, 2i] += sin(p_t * freq[i])``, ``x[t, 2i + 1] += cos(p_t * freq[i])`` in place (float32)."""
    if x.dim() != 2 or x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("add_sinusoid takes a contiguous float32 [tokens, dim]")
    tokens, dim = x.shape
    if positions.numel() != tokens or freq.numel() != (dim + 1) // 2:
        raise KernelError("add_sinusoid: one position per token and one frequency per pair of elements")
    _lib.call("pylon_add_sinusoid", _dev(x, "x", torch.float32), _dev(positions, "positions", torch.int32),
              _dev(freq, "freq", torch.float32), tokens, dim, _stream())
    return x


def add_bias_(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``x[..., i] += bias[i]`` in place; ``x`` contiguous, ``bias`` float32 of the last axis' length."""
    if not x.is_contiguous() or bias.shape != (x.shape[-1],):
        raise KernelError("add_bias_ takes a contiguous tensor and one bias per element of its last axis")
    _lib.call("pylon_add_bias", _dev(x, "x"), dtype_code(x.dtype), _dev(bias, "bias", torch.float32),
              x.numel() // x.shape[-1], x.shape[-1], _stream())
    return x


CONV_MODES = {"residual": 0, "silu": 1}


def short_conv(h: torch.Tensor, weight: torch.Tensor, state: Optional[torch.Tensor], row_start: torch.Tensor,
               row_slots: torch.Tensor, *, rows: int, max_count: int, out_dtype: torch.dtype,
               mode: str = "residual") -> torch.Tensor:
    """``h[t] + sum_j weight[:, j] * h[t - taps + 1 + j]`` per channel and request, zeros before a
    request's start.  ``state`` (float32 ``[slots, taps - 1, width]``) holds every request's last
    ``taps - 1`` inputs and is brought up to date; ``max_count`` bounds the tokens of a row.
    ``mode="silu"``: ``silu`` of the convolution alone, without the input added.  ``h`` may be
    the first columns of wider rows."""
    if h.dim() != 2 or weight.dim() != 2 or weight.shape[0] != h.shape[1] or h.stride(1) != 1:
        raise KernelError("short_conv takes h [tokens, width] and weight [width, taps]")
    tokens, width = h.shape
    taps = weight.shape[1]
    if taps > 1 and (state is None or state.dim() != 3 or state.shape[1:] != (taps - 1, width)):
        raise KernelError(f"short_conv: state must be [slots, {taps - 1}, {width}]")
    if row_start.numel() != rows + 1 or row_slots.numel() != rows:
        raise KernelError("short_conv: one start per row and one more, and one slot per row")
    out = torch.empty((tokens, width), dtype=out_dtype, device=h.device)
    _lib.call("pylon_short_conv", _dev(out, "out"), dtype_code(out_dtype), h.data_ptr(), dtype_code(h.dtype),
              _dev(weight, "weight"), dtype_code(weight.dtype), _dev(state, "state", torch.float32),
              _dev(row_start, "row_start", torch.int32), _dev(row_slots, "row_slots", torch.int32), rows,
              int(max_count), width, taps, h.stride(0) if tokens > 1 else width, CONV_MODES[mode], _stream())
    return out


RETENTION_CHUNK = 32
RETENTION_PARALLEL_BYTES = 1 << 29  # the most memory the chunks' states may take


def retention_chunk_parallel(rows: int, heads: int, dim: int, vdim: int, max_count: int,
                             units: Optional[int] = None) -> bool:
    """Whether chunked retention takes one workgroup a chunk: when one workgroup a (row, head) would
    leave most compute units idle, the rows are long enough for the two extra launches to pay, and
    the chunks' states (float32, ``dim x vdim`` a chunk and head) fit a bound."""
    units = units or _lib.compute_units()
    chunks = -(-max_count // RETENTION_CHUNK)
    return (rows * heads * 2 <= units and chunks >= 4
            and rows * heads * chunks * dim * vdim * 4 <= RETENTION_PARALLEL_BYTES)


def retention_chunked_ok(dtype: torch.dtype, *, dim: int, vdim: int, rot_dims: int) -> bool:
    """Whether the matrix-core form of retention takes this geometry (else the recurrent form does)."""
    return (dtype == torch.bfloat16 and dim % 32 == 0 and 32 <= dim <= 256 and 1 <= vdim <= 256
            and rot_dims % 2 == 0 and (dim - rot_dims) % 2 == 0)


def retention_recurrent(proj: torch.Tensor, state: torch.Tensor, decay: torch.Tensor,
                        inv_freq: Optional[torch.Tensor], positions: torch.Tensor, row_start: torch.Tensor,
                        row_slots: torch.Tensor, *, rows: int, heads: int, dim: int, vdim: int, rot_dims: int,
                        eps: float, k_scale: float, chunked: bool = False,
                        max_count: Optional[int] = None) -> torch.Tensor:
    """Retention, token by token: ``proj`` ``[tokens, 2 heads dim + 2 heads vdim]`` holds q, k, v
    and the gate side by side; ``state`` (float32 ``[slots, heads, dim, vdim]``) is read and left
    up to date.  Returns the gated, per-head normalised output ``[tokens, heads * vdim]``.
    ``chunked``: the matrix-core form for bfloat16 prompt portions, 32 tokens at a time (same
    arguments, same state).  With ``max_count`` (the most tokens a row brings) and few rows it
    takes one workgroup a chunk instead of one a (row, head): what every chunk adds to the state,
    a scan over the chunks, then every chunk's outputs (:func:`retention_chunk_parallel`)."""
    if proj.dim() != 2 or proj.shape[1] != 2 * heads * dim + 2 * heads * vdim or proj.stride(1) != 1:
        raise KernelError("retention: the projection's rows must hold q, k, v and the gate")
    tokens = proj.shape[0]
    if state.dim() != 4 or state.shape[1:] != (heads, dim, vdim):
        raise KernelError(f"retention: state must be [slots, {heads}, {dim}, {vdim}]")
    if decay.numel() != heads or positions.numel() != tokens:
        raise KernelError("retention: one decay per head and one position per token")
    if row_start.numel() != rows + 1 or row_slots.numel() != rows:
        raise KernelError("retention: one start per row and one more, and one slot per row")
    if rot_dims and (inv_freq is None or inv_freq.numel() != rot_dims // 2):
        raise KernelError("retention: inv_freq must hold rot_dims/2 frequencies")
    if not proj.is_cuda:
        raise KernelError("proj must live on the GPU; there is no CPU path")
    out = torch.empty((tokens, heads * vdim), dtype=proj.dtype, device=proj.device)
    if chunked:
        if not retention_chunked_ok(proj.dtype, dim=dim, vdim=vdim, rot_dims=rot_dims):
            raise KernelError("retention: the chunked form does not take this geometry")
        chunk_state = None
        if max_count is not None and retention_chunk_parallel(rows, heads, dim, vdim, max_count):
            chunks = -(-max_count // RETENTION_CHUNK)
            chunk_state = torch.empty((rows * heads * chunks * dim * vdim,), dtype=torch.float32, device=proj.device)
        _lib.call("pylon_retention_chunked", _dev(out, "out"), proj.data_ptr(), proj.stride(0), 0, heads * dim,
                  2 * heads * dim, 2 * heads * dim + heads * vdim, _dev(state, "state", torch.float32),
                  _dev(decay, "decay", torch.float32), _dev(inv_freq, "inv_freq", torch.float32), int(rot_dims),
                  _dev(positions, "positions", torch.int32), _dev(row_start, "row_start", torch.int32),
                  _dev(row_slots, "row_slots", torch.int32), rows, heads, dim, vdim, float(eps), float(k_scale),
                  int(max_count or 0), _dev(chunk_state, "chunk_state"),
                  0 if chunk_state is None else chunk_state.numel(), _stream())
        return out
    _lib.call("pylon_retention_recurrent", _dev(out, "out"), proj.data_ptr(), dtype_code(proj.dtype), proj.stride(0),
              0, heads * dim, 2 * heads * dim, 2 * heads * dim + heads * vdim, _dev(state, "state", torch.float32),
              _dev(decay, "decay", torch.float32), _dev(inv_freq, "inv_freq", torch.float32), int(rot_dims),
              _dev(positions, "positions", torch.int32), _dev(row_start, "row_start", torch.int32),
              _dev(row_slots, "row_slots", torch.int32), rows, heads, dim, vdim, float(eps), float(k_scale),
              _stream())
    return out


def kv_store(proj: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, slot_map: torch.Tensor, *,
             k_off: int, v_off: int, v_transposed: bool = False) -> None:
    """Copy every token's keys (``proj[t, k_off:]``) and values (``proj[t, v_off:]``) into its
    cache slot; the caches are ``[pages, page_size, kv_heads, size]`` with sizes of their own.
    With ``v_transposed`` the values go to ``[pages, kv_heads, size, page_size]``."""
    if proj.dim() != 2 or proj.stride(1) != 1 or k_cache.dim() != 4 or v_cache.dim() != 4:
        raise KernelError("kv_store takes a 2-D projection and 4-D caches")
    if k_cache.dtype != proj.dtype or v_cache.dtype != proj.dtype:
        raise KernelError("kv_store: the projection and the caches differ in dtype")
    tokens = proj.shape[0]
    if slot_map.numel() != tokens:
        raise KernelError("kv_store: one cache slot per token is required")
    k_row = k_cache.shape[2] * k_cache.shape[3]
    v_row = v_cache.shape[1] * v_cache.shape[2] if v_transposed else v_cache.shape[2] * v_cache.shape[3]
    page_size = k_cache.shape[1]
    if v_cache.numel() != k_cache.shape[0] * page_size * v_row:
        raise KernelError("kv_store: the two caches hold different numbers of slots")
    if max(k_off + k_row, v_off + v_row) > proj.shape[1]:
        raise KernelError("kv_store: keys or values lie outside the projection's rows")
    if not proj.is_cuda:
        raise KernelError("proj must live on the GPU; there is no CPU path")
    _lib.call("pylon_kv_store", _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"), proj.data_ptr(),
              dtype_code(proj.dtype), proj.stride(0), int(k_off), int(v_off), _dev(slot_map, "slot_map", torch.int32),
              tokens, k_row, v_row, page_size if v_transposed else 0, _stream())


def qkv_bias_store(proj: torch.Tensor, bias: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                   v_cache: Optional[torch.Tensor], slot_map: Optional[torch.Tensor], *, q_size: int, k_size: int,
                   v_size: int, out_dtype: torch.dtype, store: bool, v_transposed: bool = False) -> torch.Tensor:
    """A fused projection's rows ``[q | k | v]`` (its float32 sums, or rounded already; ``q`` alone for
    a run that stores nothing) get their ``bias`` (float32, a row's length, or None) and are rounded
    once to ``out_dtype``: ``q`` is returned as ``[tokens, q_size]``, keys and values go to the tokens'
    cache slots (values transposed inside their page with ``v_transposed``)."""
    if proj.dim() != 2 or proj.stride(1) != 1:
        raise KernelError("qkv_bias_store takes a 2-D projection")
    tokens, row = proj.shape
    need = q_size + (k_size + v_size if store else 0)
    if row < need or (bias is not None and bias.numel() < need):
        raise KernelError("qkv_bias_store: the projection's rows or the bias are too short")
    page_size = 0
    if store:
        if k_cache is None or v_cache is None or slot_map is None or slot_map.numel() != tokens:
            raise KernelError("qkv_bias_store: storing needs the caches and one slot per token")
        if k_cache.dtype != out_dtype or v_cache.dtype != out_dtype:
            raise KernelError("qkv_bias_store: the caches are not of the output's type")
        if k_cache.shape[2] * k_cache.shape[3] != k_size or v_cache.numel() != k_cache.shape[0] * k_cache.shape[1] * v_size:
            raise KernelError("qkv_bias_store: the caches do not match the sizes of k and v")
        page_size = k_cache.shape[1] if v_transposed else 0
    q = torch.empty((tokens, q_size), dtype=out_dtype, device=proj.device)
    _lib.call("pylon_qkv_bias_store", _dev(q, "q"), _dev(k_cache if store else None, "k_cache"),
              _dev(v_cache if store else None, "v_cache"), dtype_code(out_dtype), proj.data_ptr(),
              dtype_code(proj.dtype), proj.stride(0), _dev(bias, "bias", torch.float32),
              _dev(slot_map if store else None, "slot_map", torch.int32), tokens, q_size, k_size, v_size,
              page_size, 1 if store else 0, _stream())
    return q


def sigmoid_gate_(x: torch.Tensor, gate: torch.Tensor, *, per: int) -> torch.Tensor:
    """``x[t, i] *= sigmoid(gate[t, i // per])`` in place: ``x`` contiguous ``[tokens, n]``, ``gate``
    ``[tokens, n // per]`` of the same type (maybe columns of wider rows); ``per`` is a head's size
    for one gate per head, 1 for one per element."""
    if x.dim() != 2 or not x.is_contiguous() or gate.dim() != 2 or gate.stride(1) != 1 or gate.dtype != x.dtype:
        raise KernelError("sigmoid_gate_ takes a contiguous [tokens, n] and gates of its type")
    tokens, n = x.shape
    if per < 1 or n % per or gate.shape != (tokens, n // per):
        raise KernelError(f"sigmoid_gate_: {n} elements in groups of {per} need gates [tokens, {n // max(per, 1)}]")
    _lib.call("pylon_sigmoid_gate", _dev(x, "x"), dtype_code(x.dtype), gate.data_ptr(),
              gate.stride(0) if tokens > 1 else n // per, tokens, n, int(per), _stream())
    return x


def scaled_sum(a: torch.Tensor, a_scale: float, b: torch.Tensor, b_scale: float) -> torch.Tensor:
    """``a_scale * a + b_scale * b`` as float32 ``[tokens, dim]``; ``a`` and ``b`` are each
    ``[tokens, dim]`` or a stack ``[parts, tokens, dim]`` of float32 partial sums still to be added up."""
    shape = tuple(a.shape[-2:])
    for t in (a, b):
        if t.dim() not in (2, 3) or tuple(t.shape[-2:]) != shape or not t.is_contiguous():
            raise KernelError("scaled_sum takes two contiguous [tokens, dim] tensors or stacks of such")
        if t.dim() == 3 and t.dtype != torch.float32:
            raise KernelError("scaled_sum: a stack of partial sums is float32")
    out = torch.empty(shape, dtype=torch.float32, device=a.device)
    _lib.call("pylon_scaled_sum", _dev(out, "out"), _dev(a, "a"), dtype_code(a.dtype), a.shape[0] if a.dim() == 3 else 1,
              float(a_scale), _dev(b, "b"), dtype_code(b.dtype), b.shape[0] if b.dim() == 3 else 1, float(b_scale),
              out.numel(), _stream())
    return out


def _delta_rule_layout(dim: int, vdim: int, wide: bool):
    """``(threads a column, elements a thread)`` as the kernel lays a head over a workgroup, or None."""
    p = 1
    if wide:
        while p * 2 <= 16 and p * 2 <= dim and vdim * p * 2 <= 256:
            p *= 2
    else:
        while p < 4 and p * 2 <= dim and -(-dim // p) > 32 and vdim * p * 2 <= 1024:
            p *= 2
    r = -(-dim // p)
    while r > 64 and p * 2 <= 64 and vdim * p * 2 <= 1024:
        p *= 2
        r = -(-dim // p)
    if dim < 1 or vdim < 1 or r > 128 or vdim * p > 1024 or (r > 64 and vdim * p > 256):
        return None
    return p, r


def delta_rule_ok(dim: int, vdim: int, col_groups: int = 1) -> bool:
    """Whether :func:`delta_rule` has a layout for heads of ``dim x vdim`` whose columns are dealt to
    ``col_groups`` workgroups (the kernel's own rule)."""
    if col_groups < 1 or vdim % col_groups:
        return False
    return _delta_rule_layout(dim, vdim // col_groups, col_groups > 1) is not None


def delta_rule_col_groups(rows: int, heads: int, dim: int, vdim: int, max_count: Optional[int],
                          units: Optional[int] = None) -> int:
    """Over how many workgroups the columns of a head's state are dealt: one for steps of short rows
    (one launch, the norm inside); for rows of 64 tokens and more a power of two of at most 16 that
    divides ``vdim``, leaves every workgroup at least 16 columns and does not start more workgroups
    than twice the compute units."""
    if max_count is None or max_count < 64:
        return 1
    units = units or _lib.compute_units()
    groups = 1
    while (groups < 16 and vdim % (groups * 2) == 0 and vdim // (groups * 2) >= 16
           and rows * heads * groups * 2 <= 2 * units and delta_rule_ok(dim, vdim, groups * 2)):
        groups *= 2
    return groups


def delta_rule(qkv: torch.Tensor, proj: torch.Tensor, state: torch.Tensor, a_log: torch.Tensor,
               dt_bias: torch.Tensor, norm_weight: torch.Tensor, row_start: torch.Tensor, row_slots: torch.Tensor, *,
               rows: int, heads: int, kv_heads: int, dim: int, vdim: int, gate_off: int, beta_off: int,
               decay_off: int, eps: float, unit_eps: float, q_scale: float, out_dtype: torch.dtype,
               max_count: Optional[int] = None, col_groups: Optional[int] = None,
               chunked: Optional[bool] = None) -> torch.Tensor:
    """The gated delta rule over the rows of a step: per request and head ``S <- g S; u = beta (v -
    S^T k); S <- S + k u^T; o = S^T q``.  ``qkv`` float32 ``[tokens, 2 kv_heads dim + heads vdim]``
    holds q, k and v (after their convolution and activation); q and k become unit vectors per head
    (``unit_eps`` inside the root; q also times ``q_scale``).  ``proj`` float32 rows hold, from
    ``gate_off``, the output gate ``[heads, vdim]``, and per head the logits of ``beta`` (from
    ``beta_off``) and of the decay (from ``decay_off``): ``beta = sigmoid(b)``, ``g = exp(-exp(a_log) *
    softplus(a + dt_bias))``.  ``state`` float32 ``[slots, heads, vdim, dim]`` (the state transposed)
    is read and left up to date.  Returns ``o / rms(o) * norm_weight * silu(gate)`` as ``[tokens,
    heads * vdim]``.  ``max_count`` (the most tokens a row brings) lets long rows have the columns of
    a head's state dealt to several workgroups (:func:`delta_rule_col_groups`; ``col_groups`` says
    it outright); the results are the same numbers either way.  ``chunked``: sixteen tokens at a
    time, the rule written out over the piece, where the sizes allow; the same results up to the
    order of additions (measured no faster than token by token, and not the default)."""
    if qkv.dim() != 2 or proj.dim() != 2 or qkv.dtype != torch.float32 or proj.dtype != torch.float32 \
            or qkv.stride(1) != 1 or proj.stride(1) != 1 or qkv.shape[0] != proj.shape[0]:
        raise KernelError("delta_rule takes float32 rows of q, k, v and of the projection, one per token")
    tokens = qkv.shape[0]
    qk = kv_heads * dim
    if qkv.shape[1] < 2 * qk + heads * vdim:
        raise KernelError("delta_rule: the rows of q, k and v are too short")
    if max(gate_off + heads * vdim, beta_off + heads, decay_off + heads) > proj.shape[1] or min(gate_off, beta_off, decay_off) < 0:
        raise KernelError("delta_rule: the gate, beta or the decay lie outside the projection's rows")
    if state.dim() != 4 or state.shape[1:] != (heads, vdim, dim) or state.dtype != torch.float32 or not state.is_contiguous():
        raise KernelError(f"delta_rule: state must be float32 [slots, {heads}, {vdim}, {dim}]")
    if a_log.shape != (heads,) or dt_bias.shape != (heads,) or norm_weight.shape != (vdim,):
        raise KernelError("delta_rule: one rate and one bias per head, one norm weight per value element")
    if row_start.numel() != rows + 1 or row_slots.numel() != rows:
        raise KernelError("delta_rule: one start per row and one more, and one slot per row")
    if not delta_rule_ok(dim, vdim) or heads % kv_heads:
        raise KernelError(f"delta_rule does not take {heads} heads over {kv_heads} of {dim} x {vdim}")
    if not qkv.is_cuda:
        raise KernelError("qkv must live on the GPU; there is no CPU path")
    out = torch.empty((tokens, heads * vdim), dtype=out_dtype, device=qkv.device)
    if col_groups is None:
        col_groups = delta_rule_col_groups(rows, heads, dim, vdim, max_count)
    if not delta_rule_ok(dim, vdim, col_groups):
        raise KernelError(f"delta_rule: {vdim} columns cannot be dealt to {col_groups} workgroups")
    raw = torch.empty((tokens, heads * vdim), dtype=torch.float32, device=qkv.device) if col_groups > 1 else None
    _lib.call("pylon_delta_rule", _dev(out, "out"), dtype_code(out_dtype), heads * vdim, qkv.data_ptr(),
              qkv.stride(0) if tokens > 1 else qkv.shape[1], 0, qk, 2 * qk, proj.data_ptr(),
              proj.stride(0) if tokens > 1 else proj.shape[1], int(gate_off), int(beta_off), int(decay_off),
              _dev(a_log, "a_log", torch.float32), _dev(dt_bias, "dt_bias", torch.float32),
              _dev(norm_weight, "norm_weight", torch.float32), _dev(state, "state", torch.float32),
              _dev(row_start, "row_start", torch.int32), _dev(row_slots, "row_slots", torch.int32), rows, heads,
              kv_heads, dim, vdim, float(eps), float(unit_eps), float(q_scale), int(col_groups), _dev(raw, "raw"),
              tokens, 1 if chunked else 0, _stream())
    return out


def gated_act(gate_up: torch.Tensor, *, alpha: float, offset: float, limit: float,
              out_dtype: Optional[torch.dtype] = None, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``a(g) * (u + offset)`` for a ``[tokens, 2I]`` input holding ``g`` then ``u``, with
    ``a(g) = g * sigmoid(alpha * g)``, ``g`` capped from above at ``limit`` and ``u`` to
    ``[-limit, limit]`` (``limit <= 0``: no cap).  float32 sums in, bfloat16 out: one rounding.
    ``bias`` (float32 ``[2I]``) is added to ``g`` and ``u`` first."""
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise KernelError("gated_act takes a [tokens, 2*I] input")
    tokens, two_i = gate_up.shape
    if bias is not None and bias.shape != (two_i,):
        raise KernelError("gated_act: one bias per column of the input")
    out = torch.empty((tokens, two_i // 2), dtype=out_dtype or gate_up.dtype, device=gate_up.device)
    _lib.call("pylon_gated_act", _dev(out, "out"), dtype_code(out.dtype), _dev(gate_up, "gate_up"),
              dtype_code(gate_up.dtype), tokens, two_i // 2, float(alpha), float(offset), float(limit),
              _dev(bias, "bias", torch.float32), _stream())
    return out


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x <- cap * tanh(x / cap)`` in place (float32)."""
    _lib.call("pylon_softcap", _dev(x, "x", torch.float32), x.numel(), float(cap), _stream())
    return x


def scale_(x: torch.Tensor, factor: float) -> torch.Tensor:
    """``x *= factor`` in place (float32)."""
    _lib.call("pylon_scale", _dev(x, "x", torch.float32), x.numel(), float(factor), _stream())
    return x


DECODE_HEAD_DIMS = (64, 128, 256)
DECODE_MAX_TOKENS = 1024  # beyond this many single-token rows the prefill kernel's tiling takes over


def decode_attention_ok(q: torch.Tensor, k_cache: torch.Tensor) -> bool:
    """Whether the key-split decode kernel takes this geometry."""
    tokens, n_heads, head_dim = q.shape
    n_kv_heads = k_cache.shape[2]
    return (q.dtype == torch.bfloat16 and head_dim in DECODE_HEAD_DIMS and tokens <= DECODE_MAX_TOKENS
            and n_heads % n_kv_heads == 0 and n_heads // n_kv_heads <= 16)


def decode_splits(tokens: int, n_kv_heads: int, max_len: Optional[int], units: int = plan.UNITS) -> int:
    """Wavefronts (1, 2, 4 or 8) that share the keys of one (token, key/value head):
    ranges of about 64 keys (one batch of loads per wave) while the launch stays within a
    few thousand waves.  ``max_len`` is the most keys a workgroup gets (an upper bound
    under graph capture)."""
    waves = 8
    if tokens * n_kv_heads > units:
        # more workgroups than compute units: smaller ones run side by side (64 tokens of 140
        # keys: 13.8 us with four waves, 21.6 with eight; of 1,000 keys: 47 against 52)
        waves = 4
    while waves > 1 and tokens * n_kv_heads * waves > 16 * units:
        waves //= 2
    if max_len is not None:
        while waves > 1 and (waves // 2) * 64 >= max_len:
            waves //= 2
    return waves


def _like(q: torch.Tensor, out: Optional[torch.Tensor], name: str) -> torch.Tensor:
    if out is None:
        return torch.empty_like(q)
    if out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
        raise KernelError(f"{name}: out must be contiguous and of q's shape and dtype")
    return out


def decode_cuts(tokens: int, n_kv_heads: int, max_len: Optional[int], units: int = plan.UNITS) -> int:
    """Workgroups that share the keys of one (token, key/value head) before the waves of
    each share theirs: more than one when a few requests would otherwise occupy a fraction of
    the chip.  From 768 keys of ``max_len`` on (which may be an upper bound above the true
    lengths), each cut at least 192 keys, up to one workgroup per compute unit.  Measured on 256
    units with 8 key/value heads of 128, the launch with its merge against one workgroup per
    (token, head): 1 token of 1,000 keys 14.1 us (4 cuts) against 20.6, of 2,000 keys 14.1 (8)
    against 31, of 8,000 keys 19.1 (32) against 125; 8 tokens of 700 keys 15.2 (4) against 19.7,
    of 2,000 keys 23.6 (4) against 42; 16 tokens of 2,000 keys 35 (2) against 49.  At 500 keys one
    workgroup is within a microsecond (13.2 to 14.3 us); and once the workgroups fill the units
    (32 tokens) a cut only adds the second kernel."""
    if max_len is None or max_len < 768:
        return 1
    cuts = 1
    while cuts < 64 and tokens * n_kv_heads * cuts * 2 <= units and cuts * 2 * 192 <= max_len:
        cuts *= 2
    return cuts


def decode_launch(tokens: int, n_kv_heads: int, span: int) -> tuple:
    """(cuts, splits) for decode attention of ``tokens`` single tokens that each see at most
    ``span`` keys, on the current device."""
    units = _lib.compute_units()
    cuts = decode_cuts(tokens, n_kv_heads, span, units)
    return cuts, decode_splits(tokens * cuts, n_kv_heads, -(-span // cuts), units)


def _decode_scratch(tokens: int, n_heads: int, head_dim: int, n_cuts: int, device) -> Optional[torch.Tensor]:
    if n_cuts <= 1:
        return None
    return torch.empty((tokens * n_heads * n_cuts * (head_dim + 2),), dtype=torch.float32, device=device)


def attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     block_table: torch.Tensor, tok_row: Optional[torch.Tensor], positions: torch.Tensor, *,
                     page_size: int, window: Optional[int], scale: float, n_splits: int,
                     n_cuts: int = 1, out: Optional[torch.Tensor] = None,
                     chunk: Optional[int] = None) -> torch.Tensor:
    """Paged attention of a few bfloat16 query tokens; ``n_splits`` wavefronts share the
    keys of each (token, key/value head) and merge their partial results, after ``n_cuts``
    workgroups have shared them first (their partial results meet in a second small
    kernel).  ``tok_row`` None means token ``t`` uses row ``t`` of the block table (a
    decode-only step), which saves the kernel one dependent trip to memory."""
    if q.dim() != 3 or not decode_attention_ok(q, k_cache):
        raise KernelError("attention_decode does not take this geometry")
    tokens, n_heads, head_dim = q.shape
    pages, psize, n_kv_heads, hd = k_cache.shape
    if psize != page_size or hd != head_dim or k_cache.shape != v_cache.shape:
        raise KernelError("attention_decode: cache geometry does not match page_size/head_dim")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError("attention_decode: q and the caches differ in dtype")
    if pages * page_size >= 2 ** 31:
        raise KernelError("attention_decode: the cache holds more slots than an int32 can index")
    if positions.numel() != tokens or block_table.dim() != 2:
        raise KernelError("attention_decode: one position per token and a 2-D table are required")
    if tok_row is None:
        if block_table.shape[0] < tokens:
            raise KernelError("attention_decode: without row ids the table needs a row per token")
    elif tok_row.numel() != tokens:
        raise KernelError("attention_decode: one row id per token is required")
    out = _like(q, out, "attention_decode")
    scratch = _decode_scratch(tokens, n_heads, head_dim, n_cuts, q.device)
    _lib.call("pylon_attention_decode", _dev(out, "out"), _dev(q, "q"), _dev(k_cache, "k_cache"),
              _dev(v_cache, "v_cache"), _dev(block_table, "block_table", torch.int32), block_table.shape[1],
              _dev(tok_row, "tok_row", torch.int32), _dev(positions, "positions", torch.int32),
              tokens, n_heads, n_kv_heads, head_dim, page_size, mask_code(window, chunk), float(scale),
              int(n_splits), int(n_cuts), _dev(scratch, "scratch"), 0 if scratch is None else scratch.numel(),
              _stream())
    return out


def decode_fused_ok(qkv_dtype: torch.dtype, k_cache: torch.Tensor, *, tokens: int, n_heads: int, head_dim: int,
                    rot_dim: int) -> bool:
    """Whether the decode kernel can prepare q, k and v itself from a projection of
    ``qkv_dtype``: its geometry, and a rotation of the whole head or none."""
    n_kv_heads = k_cache.shape[2]
    return (qkv_dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and head_dim in DECODE_HEAD_DIMS
            and tokens <= DECODE_MAX_TOKENS and n_heads % n_kv_heads == 0 and n_heads // n_kv_heads <= 16
            and rot_dim in (0, head_dim))


def attention_decode_fused(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_table: torch.Tensor, tok_row: Optional[torch.Tensor], positions: torch.Tensor, *,
                           n_heads: int, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                           eps: float, inv_freq: Optional[torch.Tensor], slot_map: Optional[torch.Tensor],
                           page_size: int, window: Optional[int], scale: float, n_splits: int,
                           n_cuts: int = 1) -> torch.Tensor:
    """:func:`qkv_prepare` and :func:`attention_decode` in one launch: from the raw projection
    ``qkv`` ``[tokens, (n_heads + 2 kv_heads) * head_dim]`` (``[tokens, n_heads * head_dim]``
    when ``slot_map`` is None and nothing is stored), bfloat16, or from float32 partial sums
    ``[parts, tokens, width]`` of it, which the kernel adds in order and rounds to bfloat16
    once.  Returns ``[tokens, n_heads, head_dim]``."""
    pages, psize, n_kv_heads, head_dim = k_cache.shape
    store = slot_map is not None
    parts = 0
    if qkv.dim() == 3:
        if qkv.dtype != torch.float32 or not qkv.is_contiguous():
            raise KernelError("attention_decode_fused: partial sums come as a contiguous float32 stack")
        parts = qkv.shape[0]
    elif qkv.dim() != 2 or qkv.dtype != torch.bfloat16:
        raise KernelError("attention_decode_fused takes a bfloat16 projection or float32 partial sums of it")
    tokens, width = qkv.shape[-2:]
    if width != (n_heads + (2 * n_kv_heads if store else 0)) * head_dim:
        raise KernelError("attention_decode_fused: the projection's width does not match the heads")
    if qkv.stride(-1) != 1 or qkv.stride(-2) % 8 or qkv.data_ptr() % 16:
        raise KernelError("attention_decode_fused: the projection's rows must be contiguous and 16-byte aligned")
    if not decode_fused_ok(torch.bfloat16, k_cache, tokens=tokens, n_heads=n_heads, head_dim=head_dim,
                           rot_dim=0 if inv_freq is None else 2 * inv_freq.numel()):
        raise KernelError("attention_decode_fused does not take this geometry")
    if psize != page_size or k_cache.shape != v_cache.shape or v_cache.dtype != k_cache.dtype:
        raise KernelError("attention_decode_fused: cache geometry does not match page_size")
    if pages * page_size >= 2 ** 31:
        raise KernelError("attention_decode_fused: the cache holds more slots than an int32 can index")
    if positions.numel() != tokens or block_table.dim() != 2 or (store and slot_map.numel() != tokens):
        raise KernelError("attention_decode_fused: one position and one slot per token and a 2-D table are required")
    for name, wt in (("q_weight", q_weight), ("k_weight", k_weight)):
        if wt is not None and wt.shape != (head_dim,):
            raise KernelError(f"attention_decode_fused: {name} must have shape ({head_dim},)")
    if tok_row is None:
        if block_table.shape[0] < tokens:
            raise KernelError("attention_decode_fused: without row ids the table needs a row per token")
    elif tok_row.numel() != tokens:
        raise KernelError("attention_decode_fused: one row id per token is required")
    out = torch.empty((tokens, n_heads, head_dim), dtype=torch.bfloat16, device=qkv.device)
    scratch = _decode_scratch(tokens, n_heads, head_dim, n_cuts, qkv.device)
    _lib.call("pylon_attention_decode_fused", _dev(out, "out"), qkv.data_ptr(), qkv.stride(-2), parts,
              qkv.stride(0) if parts else 0,
              _dev(q_weight, "q_weight", torch.float32), _dev(k_weight, "k_weight", torch.float32), float(eps),
              _dev(inv_freq, "inv_freq", torch.float32), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
              _dev(slot_map, "slot_map", torch.int32), _dev(block_table, "block_table", torch.int32),
              block_table.shape[1], _dev(tok_row, "tok_row", torch.int32),
              _dev(positions, "positions", torch.int32), tokens, n_heads, n_kv_heads, head_dim, page_size,
              int(window or 0), float(scale), int(n_splits), int(n_cuts), _dev(scratch, "scratch"),
              0 if scratch is None else scratch.numel(), _stream())
    return out


PREFILL_ROWS = 128  # most (token, head) query rows one workgroup of the prefill kernel takes


def prefill_rows(tokens: int, n_heads: int, group: int) -> int:
    """Query rows per workgroup: 128 halve the traffic from LDS per matrix instruction, but a
    step with few query rows fills more of the chip with workgroups of 64 (which hold a
    group of at most 64 heads)."""
    return 128 if tokens * n_heads >= 128 * 512 or group > 64 else 64


def prefill_fold(n_kv_heads: int) -> int:
    """Tiles whose workgroups (one per tile and key/value head) fill the chip once: the unit in
    which the order of a step's tiles is folded (2,048 tokens at the Qwen3-4B geometry: 59 -> 56
    us; 4,096: 164 -> 158)."""
    return max(1, _lib.compute_units() // n_kv_heads)


PREFILL_MAX_PAGES = 4096  # block-table columns the prefill kernel keeps in LDS


def prefill_attention_ok(q: torch.Tensor, k_cache: torch.Tensor, block_table: Optional[torch.Tensor] = None) -> bool:
    tokens, n_heads, head_dim = q.shape
    n_kv_heads = k_cache.shape[2]
    return (q.dtype == torch.bfloat16 and head_dim in DECODE_HEAD_DIMS and n_heads % n_kv_heads == 0
            and n_heads // n_kv_heads <= PREFILL_ROWS
            and (block_table is None or block_table.shape[1] <= PREFILL_MAX_PAGES))


def attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_table: torch.Tensor, tiles: torch.Tensor, *, page_size: int,
                      window: Optional[int], scale: float, rows: Optional[int] = None,
                      out: Optional[torch.Tensor] = None, chunk: Optional[int] = None) -> torch.Tensor:
    """Paged causal attention of bfloat16 prompt portions on the matrix cores.  ``tiles`` is
    int32 ``[n, 4]``: first token index, token count, block-table row and first position of
    runs of at most ``rows // group`` consecutive tokens of one request; ``rows`` (64 or 128,
    default :data:`PREFILL_ROWS`) is the number of query rows a workgroup takes."""
    rows = rows or PREFILL_ROWS
    if q.dim() != 3 or not prefill_attention_ok(q, k_cache, block_table):
        raise KernelError("attention_prefill does not take this geometry")
    tokens, n_heads, head_dim = q.shape
    pages, psize, n_kv_heads, hd = k_cache.shape
    if psize != page_size or hd != head_dim or k_cache.shape != v_cache.shape:
        raise KernelError("attention_prefill: cache geometry does not match page_size/head_dim")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError("attention_prefill: q and the caches differ in dtype")
    if pages * page_size >= 2 ** 31:
        raise KernelError("attention_prefill: the cache holds more slots than an int32 can index")
    if tiles.dim() != 2 or tiles.shape[1] != 4 or block_table.dim() != 2:
        raise KernelError("attention_prefill: tiles must be [n, 4] and the block table 2-D")
    out = _like(q, out, "attention_prefill")  # rows that no tile covers are left as they are
    _lib.call("pylon_attention_prefill", _dev(out, "out"), _dev(q, "q"), _dev(k_cache, "k_cache"),
              _dev(v_cache, "v_cache"), _dev(block_table, "block_table", torch.int32), block_table.shape[1],
              _dev(tiles, "tiles", torch.int32), tiles.shape[0], n_heads, n_kv_heads, head_dim, page_size,
              mask_code(window, chunk), float(scale), int(rows), _stream())
    return out


def gemm_tiled(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: Optional[torch.dtype] = None,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` with float accumulation on the vector units (no matrix cores)."""
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise KernelError(f"gemm: cannot multiply {tuple(x.shape)} by the transpose of {tuple(weight.shape)}")
    m, k = x.shape
    n = weight.shape[0]
    out_dtype = out_dtype or x.dtype
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    elif out.shape != (m, n):
        raise KernelError("gemm: out has the wrong shape")
    if x.stride(1) != 1 or weight.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: rows must be contiguous")
    for name, t in (("x", x), ("weight", weight), ("out", out)):
        if not t.is_cuda:
            raise KernelError(f"gemm: {name} must live on the GPU; there is no CPU path")
    _lib.call("pylon_gemm_tiled", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), dtype_code(x.dtype),
              weight.data_ptr(), dtype_code(weight.dtype), m, n, k, x.stride(0), weight.stride(0),
              out.stride(0), _stream())
    return out


SKINNY_ROWS = plan.FEW_ROWS    # one tile of rows of x
STREAM_ROWS = plan.STREAM_ROWS  # most rows of x a workgroup of a weight-streaming kernel takes
SPLIT_ROWS = plan.SPLIT_ROWS    # most rows the rows kernel takes, as two halves


def _streaming_ok(x: torch.Tensor, weight: torch.Tensor, rows: int) -> bool:
    """Operands a weight-streaming kernel takes: bfloat16, at most ``rows`` rows of x, rows of
    multiples of 8 elements at 16-byte aligned addresses."""
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and 0 < x.shape[0] <= rows
            and weight.shape[1] % 8 == 0 and weight.stride(0) % 8 == 0 and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def gemm_skinny(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: torch.dtype = torch.bfloat16,
                parts: int = 1, glu: bool = False,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` for at most 64 rows of bfloat16 ``x``, streaming ``weight`` once.

    ``parts > 1`` cuts K into that many ranges and returns float32 partial results
    ``[parts, M, N]`` for the consumer to add.  ``glu``: ``weight`` is a fused
    ``[2N, K]`` gate/up matrix and the result is ``silu(x @ gate.T) * (x @ up.T)``.
    """
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise KernelError(f"gemm_skinny: cannot multiply {tuple(x.shape)} by the transpose of {tuple(weight.shape)}")
    m, k = x.shape
    n = weight.shape[0]
    if glu:
        if n % 2:
            raise KernelError("gemm_skinny: a fused gate/up matrix has an even number of rows")
        n //= 2
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise KernelError("gemm_skinny takes bfloat16 operands")
    if not (x.is_cuda and weight.is_cuda) or x.stride(1) != 1 or weight.stride(1) != 1:
        raise KernelError("gemm_skinny: operands must be on the GPU with contiguous rows")
    shape = (parts, m, n) if parts > 1 else (m, n)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32 if parts > 1 else out_dtype, device=x.device)
    elif tuple(out.shape) != shape or out.dtype != (torch.float32 if parts > 1 else out_dtype) \
            or not out.is_cuda or not out.is_contiguous():
        raise KernelError(f"gemm_skinny: out must be contiguous, on the GPU and of shape {shape}")
    _lib.call("pylon_gemm_skinny", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), weight.data_ptr(),
              m, n, k, x.stride(0), weight.stride(0), n, parts, m * n, 1 if glu else 0, _stream())
    return out


def gemm_rows(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: torch.dtype = torch.bfloat16,
              parts: int = 1, col_tiles: int = 1, glu: bool = False, waves: int = 0, cols: int = 0,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` for at most 128 rows of bfloat16 ``x``: the rows of ``x`` pass through
    LDS once per workgroup of up to 64 (``col_tiles=1``) or 128 (``col_tiles=2``) columns and
    ``weight`` is streamed once (beyond 64 rows each half of the rows has workgroups of its
    own, and two that take the same columns run side by side).  ``parts > 1`` cuts K into that many ranges and returns
    float32 partial results ``[parts, M, N]`` for the consumer to add.  ``glu``: ``weight`` is
    a fused ``[2N, K]`` gate/up matrix and the result is ``silu(x @ gate.T) * (x @ up.T)``,
    rounded once.  ``waves``: wavefronts per workgroup, 4 or 2 (0: the kernel's choice);
    ``cols``: columns per workgroup (0: the kernel's choice, an equal share for every
    workgroup of whole rounds over the compute units where that pays).  The sums depend on
    neither."""
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise KernelError(f"gemm_rows: cannot multiply {tuple(x.shape)} by the transpose of {tuple(weight.shape)}")
    m, k = x.shape
    n = weight.shape[0]
    if glu:
        if n % 2:
            raise KernelError("gemm_rows: a fused gate/up matrix has an even number of rows")
        n //= 2
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise KernelError("gemm_rows takes bfloat16 operands")
    if not (x.is_cuda and weight.is_cuda) or x.stride(1) != 1 or weight.stride(1) != 1:
        raise KernelError("gemm_rows: operands must be on the GPU with contiguous rows")
    shape = (parts, m, n) if parts > 1 else (m, n)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32 if parts > 1 else out_dtype, device=x.device)
    elif tuple(out.shape) != shape or out.dtype != (torch.float32 if parts > 1 else out_dtype) \
            or not out.is_cuda or not out.is_contiguous():
        raise KernelError(f"gemm_rows: out must be contiguous, on the GPU and of shape {shape}")
    _lib.call("pylon_gemm_rows", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), weight.data_ptr(),
              m, n, k, x.stride(0), weight.stride(0), n, parts, m * n, int(col_tiles), 1 if glu else 0, int(waves),
              int(cols), _stream())
    return out


def _library_float(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` of bfloat16 operands as float32: the library's product with a float32
    result, that is its float32 sums before any rounding."""
    if out is None:
        return torch.mm(x, weight.t(), out_dtype=torch.float32)
    return torch.mm(x, weight.t(), out_dtype=torch.float32, out=out)


def linear(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: Optional[torch.dtype] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` (into ``out`` if given: contiguous, of the result's shape and type).

    bfloat16 by bfloat16: up to 64 rows go to a weight-streaming kernel where one is faster
    (:func:`plan.plan_projection`), more rows to the library matrix product (as the
    reference's ``nn.Linear`` does).  With a bfloat16 result the float32 sums are rounded once
    either way; with a float32 result (the logits) they come back unrounded either way (the
    library then writes its float32 sums): what a request's logits are rounded to does not
    depend on how many rows share its step.  Every pairing that involves float32 operands runs
    on the exact tiled kernel, which never uses a reduced-precision matrix mode.
    """
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
        if not x.is_cuda:
            raise KernelError("linear: operands must live on the GPU; there is no CPU path")
        if _streaming_ok(x, weight, STREAM_ROWS):
            choice = plan.plan_projection(x.shape[0], *weight.shape)  # no rule of it counts compute units
            if choice.kernel == "rows":
                return gemm_rows(x, weight, out_dtype=out_dtype, col_tiles=choice.col_tiles, out=out)
            if choice.kernel == "skinny":
                return gemm_skinny(x, weight, out_dtype=out_dtype, out=out)
        if out_dtype == torch.float32:
            return _library_float(x, weight, out)
        y = torch.nn.functional.linear(x, weight)
        y = y if out_dtype == torch.bfloat16 else y.to(out_dtype)
        return y if out is None else out.copy_(y)
    return gemm_tiled(x, weight, out_dtype=out_dtype, out=out)


def linear_summed_later(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: torch.dtype) -> torch.Tensor:
    """``x @ weight.T`` for a consumer that takes either the product in ``out_dtype`` or float32
    partial sums ``[parts, M, N]`` of it, to be added in order and rounded to ``out_dtype`` once
    (:func:`attention_decode_fused` does): up to 128 bfloat16 rows the weight-streaming
    kernel with K cut over workgroups (:func:`plan.plan_summed_later`), else :func:`linear`."""
    if out_dtype == torch.bfloat16 and _streaming_ok(x, weight, SPLIT_ROWS):
        choice = plan.plan_summed_later(x.shape[0], *weight.shape, units=_lib.compute_units())
        if choice.kernel == "rows" and choice.parts > 1:
            return gemm_rows(x, weight, out_dtype=torch.float32, parts=choice.parts, col_tiles=choice.col_tiles)
    return linear(x, weight, out_dtype=out_dtype)


def linear_for_residual(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: torch.dtype) -> torch.Tensor:
    """A product whose result is about to be added to the float32 residual stream.  For up
    to 128 bfloat16 rows it comes back as unrounded float32 sums, which the fused residual norm
    adds: partial sums ``[parts, M, N]`` of a streaming kernel (K cut over workgroups), or,
    from 17 rows on for a matrix at which the library is faster, the library's float32
    result (:func:`plan.plan_residual`).  For more rows (prompt portions) it is the library's
    product rounded once to bfloat16."""
    if _streaming_ok(x, weight, SPLIT_ROWS):
        choice = plan.plan_residual(x.shape[0], *weight.shape, units=_lib.compute_units())
        if choice.kernel == "rows":
            return gemm_rows(x, weight, out_dtype=torch.float32, parts=choice.parts, col_tiles=choice.col_tiles)
        if choice.kernel == "skinny":
            return gemm_skinny(x, weight, out_dtype=torch.float32, parts=choice.parts)
        return _library_float(x, weight)
    return linear(x, weight, out_dtype=out_dtype)


def linear_glu(x: torch.Tensor, gate_up: torch.Tensor, *, out_dtype: torch.dtype) -> torch.Tensor:
    """``silu(x @ gate.T) * (x @ up.T)`` for a fused ``[2I, K]`` gate/up matrix.  Up to 128
    bfloat16 rows: the activation works on the float32 sums and its result is rounded once
    (in a streaming kernel's epilogue; or, where the library is faster and beyond 64 rows,
    from its float32 result: :func:`plan.plan_gated`).  More rows (prompt portions): the
    library's product rounded to bfloat16 first."""
    if _streaming_ok(x, gate_up, SPLIT_ROWS) and x.is_cuda and gate_up.shape[0] % 2 == 0:
        choice = plan.plan_gated(x.shape[0], gate_up.shape[0] // 2, gate_up.shape[1], gate_up.stride(0))
        if choice.kernel == "rows":
            return gemm_rows(x, gate_up, out_dtype=out_dtype, glu=True)
        if choice.kernel == "skinny":
            return gemm_skinny(x, gate_up, out_dtype=out_dtype, glu=True)
        return silu_gate(_library_float(x, gate_up), out_dtype=out_dtype)
    return silu_gate(linear(x, gate_up, out_dtype=out_dtype))


def _chosen_args(rows: int, chosen: Optional[torch.Tensor], place: Optional[torch.Tensor]):
    """The optional table that also receives the chosen ids: ``chosen[place[r]] = id``."""
    if chosen is None and place is None:
        return None, None
    if chosen is None or place is None:
        raise KernelError("chosen and place go together")
    if place.numel() != rows:
        raise KernelError("place must have one index per row")
    return _dev(chosen, "chosen", torch.int32), _dev(place, "place", torch.int32)


def _ids_out(rows: int, device, out: Optional[torch.Tensor]) -> torch.Tensor:
    if out is None:
        return torch.empty((rows,), dtype=torch.int32, device=device)
    if out.shape != (rows,) or out.dtype != torch.int32 or not out.is_cuda:
        raise KernelError("out must be int32 [rows] on the GPU")
    return out


_argmax_scratch: dict = {}


def _argmax_partials(rows: int, device: torch.device) -> torch.Tensor:
    """The first launch leaves up to 64 partial results of 8 bytes per row for the second: one
    buffer per device, kept and grown, so that a serving loop allocates nothing per step.
    Calls on one stream follow each other; callers on other streams bring their own order."""
    need = max(rows, 1) * 64 * 8
    have = _argmax_scratch.get(device)
    if have is None or have.numel() < need:
        have = torch.empty((max(need, 256 * 64 * 8),), dtype=torch.uint8, device=device)
        _argmax_scratch[device] = have
    return have


def argmax(logits: torch.Tensor, *, out: Optional[torch.Tensor] = None,
           chosen: Optional[torch.Tensor] = None, place: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The index of each row's largest logit (the lowest among equals); with ``chosen`` and
    ``place`` the ids are also written to ``chosen[place[r]]``."""
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax takes [rows, vocab] logits with contiguous rows")
    rows, vocab = logits.shape
    if not logits.is_cuda or logits.dtype != torch.float32:
        raise KernelError("argmax takes float32 logits on the GPU")
    out = _ids_out(rows, logits.device, out)
    chosen_ptr, place_ptr = _chosen_args(rows, chosen, place)
    scratch = _argmax_partials(rows, logits.device)
    _lib.call("pylon_argmax", out.data_ptr(), logits.data_ptr(), rows, vocab, logits.stride(0),
              chosen_ptr, place_ptr, scratch.data_ptr(), scratch.numel(), _stream())
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, *, out: Optional[torch.Tensor] = None,
           chosen: Optional[torch.Tensor] = None, place: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row; rows with temperature 0 take the argmax.  ``chosen`` and ``place``
    as for :func:`argmax`."""
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample takes [rows, vocab] logits with contiguous rows")
    rows, vocab = logits.shape
    if not logits.is_cuda or logits.dtype != torch.float32:
        raise KernelError("sample takes float32 logits on the GPU")
    for name, t in (("temperature", temperature), ("top_p", top_p), ("uniform", uniform)):
        if t.numel() != rows:
            raise KernelError(f"sample: {name} must have one value per row")
    out = _ids_out(rows, logits.device, out)
    chosen_ptr, place_ptr = _chosen_args(rows, chosen, place)
    _lib.call("pylon_sample", out.data_ptr(), logits.data_ptr(), rows, vocab, logits.stride(0),
              _dev(temperature, "temperature", torch.float32), _dev(top_p, "top_p", torch.float32),
              _dev(uniform, "uniform", torch.float32), chosen_ptr, place_ptr, _stream())
    return out


def qkv_prepare_wide(qkv: torch.Tensor, q_out: torch.Tensor, k_cache: Optional[torch.Tensor],
                     v_cache: Optional[torch.Tensor], *, n_heads: int, n_kv_heads: int, head_dim: int, v_dim: int,
                     q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                     inv_freq: Optional[torch.Tensor], rot_dim: int, interleaved: bool,
                     positions: Optional[torch.Tensor], slot_map: Optional[torch.Tensor], store_kv: bool,
                     per_head: bool = False, rot_scale: float = 1.0, values_from_keys: bool = False,
                     v_transposed: bool = False) -> None:
    """q/k/v preparation with norms over whole projections: ``q_weight`` (float32, all heads of q
    side by side) and ``k_weight`` norm the whole q row and the whole k row of a token (None: no
    norm); the first ``rot_dim`` elements of every head of q and k are rotated by ``position *
    inv_freq[i]``, pairing neighbours (``interleaved``) or halves; q goes to ``q_out``, k and v
    (heads of ``v_dim`` elements) into the tokens' cache slots.  ``per_head``: the norms run head
    by head with weights of ``head_dim`` elements.  ``rot_scale`` multiplies every cosine and
    sine.  ``values_from_keys``: there are no value columns; the values are the keys as projected,
    before norm and rotation (``v_dim`` is then ``head_dim``).  The rows of ``qkv`` may be wider
    than q, k and v together (further columns of a fused projection are left alone).
    ``v_transposed``: the values go into their pages as ``[pages, kv_heads, v_dim, page_size]``
    (``v_cache`` is given in that shape; the page's size is the keys' cache's)."""
    if qkv.dim() != 2 or qkv.stride(1) != 1:
        raise KernelError("qkv_prepare_wide takes a 2-D projection output with contiguous rows")
    tokens, width = qkv.shape
    q_size, k_size, v_size = n_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * v_dim
    if values_from_keys and v_dim != head_dim:
        raise KernelError("qkv_prepare_wide: values that are the keys have the keys' size")
    v_offset = q_size if values_from_keys else q_size + k_size
    if width < q_size + (max(k_size, v_offset - q_size + v_size) if store_kv else 0):
        raise KernelError(f"qkv_prepare_wide: projection width {width} does not match the heads")
    if q_out.shape != (tokens, n_heads, head_dim) or q_out.dtype != qkv.dtype:
        raise KernelError("qkv_prepare_wide: q_out has the wrong shape or dtype")
    if q_weight is not None and q_weight.shape != ((head_dim,) if per_head else (q_size,)):
        raise KernelError(f"qkv_prepare_wide: q_weight must have shape ({head_dim if per_head else q_size},)")
    if k_weight is not None and k_weight.shape != ((head_dim,) if per_head else (k_size,)):
        raise KernelError(f"qkv_prepare_wide: k_weight must have shape ({head_dim if per_head else k_size},)")
    if rot_dim and (inv_freq is None or inv_freq.numel() != rot_dim // 2 or positions is None
                    or positions.numel() != tokens):
        raise KernelError("qkv_prepare_wide: a rotation needs rot_dim/2 frequencies and one position per token")
    if store_kv:
        if k_cache is None or v_cache is None or slot_map is None or slot_map.numel() != tokens:
            raise KernelError("qkv_prepare_wide: storing needs k_cache, v_cache and one slot per token")
        if k_cache.dtype != qkv.dtype or k_cache.shape[-2:] != (n_kv_heads, head_dim):
            raise KernelError(f"qkv_prepare_wide: k_cache must be [..., {n_kv_heads}, {head_dim}] of {qkv.dtype}")
        v_tail = tuple(v_cache.shape[-3:-1]) if v_transposed else tuple(v_cache.shape[-2:])
        if v_cache.dtype != qkv.dtype or v_tail != (n_kv_heads, v_dim) or \
                (v_transposed and (k_cache.dim() != 4 or v_cache.shape[-1] != k_cache.shape[1])):
            raise KernelError(f"qkv_prepare_wide: v_cache must be [..., {n_kv_heads}, {v_dim}] of {qkv.dtype} "
                              "(or, transposed, [pages, kv_heads, v_dim, page_size])")
    if not qkv.is_cuda:
        raise KernelError("qkv must live on the GPU; there is no CPU path")
    _lib.call("pylon_qkv_prepare_wide", _dev(q_out, "q_out"), _dev(k_cache if store_kv else None, "k_cache"),
              _dev(v_cache if store_kv else None, "v_cache"), qkv.data_ptr(), dtype_code(qkv.dtype), qkv.stride(0),
              _dev(q_weight, "q_weight", torch.float32), _dev(k_weight, "k_weight", torch.float32), float(eps),
              _dev(inv_freq, "inv_freq", torch.float32), int(rot_dim), 1 if interleaved else 0,
              _dev(positions, "positions", torch.int32), _dev(slot_map if store_kv else None, "slot_map", torch.int32),
              tokens, n_heads, n_kv_heads, head_dim, v_dim, 1 if store_kv else 0, 1 if per_head else 0,
              float(rot_scale), int(v_offset), int(k_cache.shape[1]) if (store_kv and v_transposed) else 0, _stream())


def latent_prepare(down: torch.Tensor, cache: Optional[torch.Tensor], slot_map: Optional[torch.Tensor], *,
                   q_rank: int, kv_rank: int, n_gate: int, q_weight: torch.Tensor, c_weight: torch.Tensor,
                   eps: float, out_dtype: torch.dtype):
    """From the float32 sums ``down`` ``[tokens, q_rank + kv_rank + n_gate]`` of a fused down
    projection: the normed query latent ``[tokens, q_rank]`` in ``out_dtype``, the normed key/value
    latent into ``cache`` (``[..., kv_rank]`` of ``out_dtype``) at the tokens' slots (``cache``
    None: nothing is stored), and ``sigmoid`` of the last ``n_gate`` numbers as float32
    ``[tokens, n_gate]`` (None without gates).  Both norms in float32."""
    if down.dim() != 2 or down.dtype != torch.float32 or down.stride(1) != 1:
        raise KernelError("latent_prepare takes float32 sums [tokens, width] with contiguous rows")
    tokens, width = down.shape
    if width != q_rank + kv_rank + n_gate:
        raise KernelError(f"latent_prepare: rows of {width} numbers, expected {q_rank + kv_rank + n_gate}")
    if q_weight.shape != (q_rank,) or c_weight.shape != (kv_rank,):
        raise KernelError("latent_prepare: the norms' weights have the latents' sizes")
    store = cache is not None
    if store and (slot_map is None or slot_map.numel() != tokens or cache.dtype != out_dtype
                  or cache.shape[-1] != kv_rank or not cache.is_contiguous()):
        raise KernelError("latent_prepare: the cache must be [..., kv_rank] of the output type, with one slot per token")
    q_latent = torch.empty((tokens, q_rank), dtype=out_dtype, device=down.device)
    gate = torch.empty((tokens, n_gate), dtype=torch.float32, device=down.device) if n_gate else None
    _lib.call("pylon_latent_prepare", _dev(q_latent, "q_latent"), _dev(cache, "cache"), _dev(gate, "gate"),
              _dev(down, "down") if down.is_contiguous() else down.data_ptr(), down.stride(0), dtype_code(out_dtype),
              _dev(q_weight, "q_weight", torch.float32), _dev(c_weight, "c_weight", torch.float32), float(eps),
              _dev(slot_map if store else None, "slot_map", torch.int32), tokens, q_rank, kv_rank, n_gate,
              1 if store else 0, _stream())
    return q_latent, gate


HEAD_PROJECT_ROWS = 64  # up to this many tokens the per-head products of bfloat16 run on the engine's own kernel


def head_project(x: torch.Tensor, m: torch.Tensor, *, gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t, h] = gate[t, h] * x[t, h] @ m[h]`` for ``x`` ``[tokens, heads, n_in]`` (the heads of
    a row side by side, rows maybe apart) and ``m`` ``[heads, n_in, n_out]``; ``gate`` float32
    ``[tokens, heads]`` or None.  float32 operands and up to 64 bfloat16 tokens: the engine's
    kernel (float sums in the order of ``n_in``, one rounding); more bfloat16 tokens: the
    library's batched product, then the gate."""
    if x.dim() != 3 or m.dim() != 3 or m.shape[0] != x.shape[1] or m.shape[1] != x.shape[2]:
        raise KernelError(f"head_project: cannot multiply {tuple(x.shape)} head by head by {tuple(m.shape)}")
    tokens, heads, n_in = x.shape
    n_out = m.shape[2]
    if x.stride(2) != 1 or x.stride(1) != n_in or not m.is_contiguous() or not x.is_cuda:
        raise KernelError("head_project: the heads of a row lie side by side, m is contiguous, both on the GPU")
    if gate is not None and (gate.shape != (tokens, heads) or gate.dtype != torch.float32):
        raise KernelError("head_project: gate must be float32 [tokens, heads]")
    if x.dtype == torch.bfloat16 and m.dtype == torch.bfloat16 and tokens > HEAD_PROJECT_ROWS:
        out = torch.empty((tokens, heads, n_out), dtype=x.dtype, device=x.device)
        torch.bmm(x.transpose(0, 1), m, out=out.transpose(0, 1))
        if gate is not None:
            _lib.call("pylon_gate_heads", _dev(out, "out"), dtype_code(out.dtype), _dev(gate, "gate", torch.float32),
                      tokens * heads, n_out, _stream())
        return out
    out = torch.empty((tokens, heads, n_out), dtype=x.dtype, device=x.device)
    _lib.call("pylon_head_project", _dev(out, "out"), x.data_ptr(), dtype_code(x.dtype),
              x.stride(0) if tokens > 1 else heads * n_in, _dev(m, "m"), dtype_code(m.dtype),
              _dev(gate, "gate", torch.float32), tokens, heads, n_in, n_out, _stream())
    return out


ROUTE_SCORINGS = {"top_softmax": 0, "sigmoid": 1}


def route_top(logits: torch.Tensor, bias: Optional[torch.Tensor], *, n_experts: int, top: int,
              shared_gate: bool, scoring: str = "top_softmax"):
    """From float32 router logits ``[tokens, n_experts (+ 1 with shared_gate)]``: the ``top``
    experts with the largest ``logit + bias`` per token (int32 ``[tokens, top]``, the lower index
    among equals), the softmax over those alone (float32 ``[tokens, top]``), and ``sigmoid`` of the
    last column (float32 ``[tokens]``, or None).  ``scoring="sigmoid"``: the weights are the chosen
    experts' own ``sigmoid(logit + bias)``, as they are."""
    if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("route_top takes float32 logits [tokens, experts]")
    tokens = logits.shape[0]
    if logits.shape[1] != n_experts + (1 if shared_gate else 0):
        raise KernelError("route_top: the logits' columns do not match the experts")
    if bias is not None and bias.shape != (n_experts,):
        raise KernelError("route_top: one bias per expert")
    experts = torch.empty((tokens, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((tokens, top), dtype=torch.float32, device=logits.device)
    gate = torch.empty((tokens,), dtype=torch.float32, device=logits.device) if shared_gate else None
    _lib.call("pylon_route_top", _dev(experts, "experts"), _dev(weights, "weights"), _dev(gate, "gate"),
              logits.data_ptr(), logits.stride(0), _dev(bias, "bias", torch.float32), tokens, n_experts, top,
              ROUTE_SCORINGS[scoring], _stream())
    return experts, weights, gate


def route_scored(logits: torch.Tensor, correction: Optional[torch.Tensor], *, n_experts: int, top: int,
                 groups: int = 1, keep: int = 1, scale: float = 1.0):
    """From float32 router logits ``[tokens, outputs]``, of which the first ``n_experts`` are experts
    and the others identity experts: scores are the softmax over all outputs; ``correction`` (float32
    ``[outputs]``) is added for the choice only; the outputs form ``groups`` equal groups of
    neighbours, and only the ``keep`` groups with the largest corrected score may be chosen from;
    the ``top`` largest corrected scores are taken (the lower index among equals).  Returns the
    chosen outputs (int32 ``[tokens, top]``; an identity keeps its index ``>= n_experts``), their
    weights ``score * scale`` (float32 ``[tokens, top]``, zero for an identity) and the sum of the
    chosen identities' weights (float32 ``[tokens]``; None if every output is an expert)."""
    if logits.dim() != 2 or logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise KernelError("route_scored takes float32 logits [tokens, outputs]")
    tokens, outputs = logits.shape
    if correction is not None and correction.shape != (outputs,):
        raise KernelError("route_scored: one correction per router output")
    experts = torch.empty((tokens, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((tokens, top), dtype=torch.float32, device=logits.device)
    identity = torch.empty((tokens,), dtype=torch.float32, device=logits.device) if outputs > n_experts else None
    _lib.call("pylon_route_scored", _dev(experts, "experts"), _dev(weights, "weights"), _dev(identity, "identity"),
              logits.data_ptr(), logits.stride(0), _dev(correction, "correction", torch.float32), tokens, outputs,
              n_experts, top, int(groups), int(keep), float(scale), _stream())
    return experts, weights, identity


EXPERT_ACTS = {"silu_gated": 0, "relu2": 1}  # silu(W_gate x) * (W_up x); relu(W_up x)^2


def expert_gate_up(x: torch.Tensor, gate_up: torch.Tensor, experts: torch.Tensor, *, n_experts: int,
                   ff: int, act: str = "silu_gated", input_weights: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(W_gate[e] x_t) * (W_up[e] x_t)`` for every token and each of its chosen experts:
    ``gate_up`` is ``[n_experts * 2 ff, width]`` (an expert's gate rows, then its up rows);
    returns ``[tokens * top, ff]`` of ``x``'s type, float sums rounded once.  ``act="relu2"``: plain
    experts, ``relu(W_up[e] x_t)^2`` with the matrix ``[n_experts * ff, width]``.  A choice of
    ``n_experts`` or more (an identity) is passed over: its rows of the result are not written.
    ``input_weights`` (float32 ``[tokens, top]``): a choice's expert works on ``x_t`` times the
    choice's weight (formed in float32)."""
    tokens, width = x.shape
    top = experts.shape[1]
    if input_weights is not None and (input_weights.shape != (tokens, top) or input_weights.dtype != torch.float32
                                      or not input_weights.is_contiguous()):
        raise KernelError("expert_gate_up: input_weights must be float32 [tokens, top]")
    per_expert = 2 * ff if act == "silu_gated" else ff
    if gate_up.shape != (n_experts * per_expert, width) or gate_up.stride(1) != 1 or x.stride(1) != 1:
        raise KernelError(f"expert_gate_up: the experts' matrix must be [experts * {per_expert}, width]")
    if experts.shape[0] != tokens or experts.dtype != torch.int32 or not experts.is_contiguous():
        raise KernelError("expert_gate_up: experts must be int32 [tokens, top]")
    hidden = torch.empty((tokens * top, ff), dtype=x.dtype, device=x.device)
    _lib.call("pylon_expert_gate_up", _dev(hidden, "hidden"), x.data_ptr(), dtype_code(x.dtype), x.stride(0),
              gate_up.data_ptr(), dtype_code(gate_up.dtype), gate_up.stride(0), _dev(experts, "experts"), tokens, top,
              ff, width, EXPERT_ACTS[act], n_experts, _dev(input_weights, "input_weights", torch.float32), _stream())
    return hidden


def expert_down(hidden: torch.Tensor, down: torch.Tensor, experts: torch.Tensor, weights: torch.Tensor, *,
                n_experts: int, width: int, shared: Optional[torch.Tensor] = None,
                shared_gate: Optional[torch.Tensor] = None, identity_x: Optional[torch.Tensor] = None,
                identity_weight: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 ``[tokens, width]``: ``sum_s weights[t, s] W_down[e_s] hidden[(t, s)]`` with ``down``
    ``[n_experts * width, ff]``, plus ``shared_gate[t] * shared[t]`` (``shared`` float32
    ``[tokens, width]``; without the gate it is added as it is), plus ``identity_weight[t] *
    identity_x[t]`` (the identity experts' share: the token's input, of ``hidden``'s type).  Choices
    of ``n_experts`` or more are passed over."""
    tokens, top = experts.shape
    ff = hidden.shape[1]
    if hidden.shape[0] != tokens * top or not hidden.is_contiguous():
        raise KernelError("expert_down: hidden must be [tokens * top, ff]")
    if down.shape != (n_experts * width, ff) or down.stride(1) != 1:
        raise KernelError("expert_down: the experts' matrix must be [experts * width, ff]")
    if weights.shape != (tokens, top) or weights.dtype != torch.float32:
        raise KernelError("expert_down: weights must be float32 [tokens, top]")
    if shared is not None and (shared.shape != (tokens, width) or shared.dtype != torch.float32):
        raise KernelError("expert_down: the shared expert's output must be float32 [tokens, width]")
    if shared_gate is not None and (shared is None or shared_gate.numel() != tokens):
        raise KernelError("expert_down: one gate per token, and only with a shared output")
    if (identity_x is None) != (identity_weight is None):
        raise KernelError("expert_down: the identities' inputs and weights go together")
    if identity_x is not None and (identity_x.shape != (tokens, width) or identity_x.dtype != hidden.dtype
                                   or identity_x.stride(1) != 1 or identity_weight.numel() != tokens):
        raise KernelError("expert_down: the identities' input must be [tokens, width] of the hidden activations' type")
    out = torch.empty((tokens, width), dtype=torch.float32, device=hidden.device)
    _lib.call("pylon_expert_down", _dev(out, "out"), _dev(hidden, "hidden"), dtype_code(hidden.dtype),
              down.data_ptr(), dtype_code(down.dtype), down.stride(0), _dev(experts, "experts", torch.int32),
              _dev(weights, "weights", torch.float32), _dev(shared, "shared", torch.float32),
              _dev(shared_gate, "shared_gate", torch.float32), tokens, top, ff, width, n_experts,
              0 if identity_x is None else identity_x.data_ptr(), 0 if identity_x is None else identity_x.stride(0),
              _dev(identity_weight, "identity_weight", torch.float32), _stream())
    return out


GROUPED_FROM = 33  # from this many tokens of a step on, the experts' products run expert by expert on the matrix cores


def experts_grouped_ok(x: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor) -> bool:
    """Whether :func:`experts_grouped` takes these operands: bfloat16 throughout, rows of multiples
    of 8 elements at 16-byte aligned addresses."""
    return (x.dtype == torch.bfloat16 and gate_up.dtype == torch.bfloat16 and down.dtype == torch.bfloat16
            and x.shape[1] % 8 == 0 and down.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and x.stride(1) == 1
            and gate_up.stride(0) % 8 == 0 and down.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and gate_up.data_ptr() % 16 == 0 and down.data_ptr() % 16 == 0)


def experts_grouped(x: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, experts: torch.Tensor,
                    weights: torch.Tensor, *, n_experts: int, ff: int, shared: Optional[torch.Tensor] = None,
                    shared_gate: Optional[torch.Tensor] = None, act: str = "silu_gated",
                    identity_weight: Optional[torch.Tensor] = None, weight_on_input: bool = False) -> torch.Tensor:
    """What :func:`expert_gate_up` and :func:`expert_down` compute, for many bfloat16 tokens: the
    (token, choice) pairs are sorted by expert on the device (nothing is read back), every expert's
    pairs go through its gate/up and its down matrix as tiles of 64 rows on the matrix cores, and
    the results return to their tokens weighted, in the order of the token's choices.  float32
    ``[tokens, width]``.  ``act`` as for :func:`expert_gate_up`.  Choices of ``n_experts`` or more
    (identity experts) sort behind every expert's pairs and run through no matrix; with
    ``identity_weight`` (float32 ``[tokens]``) ``identity_weight[t] * x[t]`` is added for them.
    ``weight_on_input``: a choice's weight multiplies its expert's input instead of its output
    (gated experts: the gate's and the up's float32 sums are scaled before the activation, which
    is the product of the scaled input because the two products are linear)."""
    tokens, width = x.shape
    top = experts.shape[1]
    pairs = tokens * top
    if not experts_grouped_ok(x, gate_up, down):
        raise KernelError("experts_grouped does not take these operands")
    per_expert = 2 * ff if act == "silu_gated" else ff
    if gate_up.shape != (n_experts * per_expert, width) or down.shape != (n_experts * width, ff):
        raise KernelError(f"experts_grouped: the experts' matrices must be [experts * {per_expert}, width] and [experts * width, ff]")
    flat = experts.reshape(-1).long()
    order = torch.argsort(flat, stable=True)  # sorted place -> pair
    bounds = torch.arange(n_experts + 1, device=x.device)
    offsets = torch.searchsorted(flat[order], bounds).to(torch.int32)
    rows = (order // top).to(torch.int32)  # sorted place -> token
    place = torch.empty_like(order).scatter_(0, order, torch.arange(pairs, device=x.device)).to(torch.int32)
    hidden = torch.empty((pairs, ff), dtype=torch.bfloat16, device=x.device)
    row_scale = None
    if weight_on_input:
        if act != "silu_gated":
            raise KernelError("experts_grouped: weights on the input go with gated experts")
        row_scale = weights.reshape(-1)[order].contiguous()  # sorted place -> the pair's weight
        weights = torch.ones_like(weights)
    _lib.call("pylon_grouped_gate_up", _dev(hidden, "hidden"), x.data_ptr(), x.stride(0), _dev(rows, "rows"),
              gate_up.data_ptr(), gate_up.stride(0), _dev(offsets, "offsets"), pairs, n_experts, ff, width, tokens,
              EXPERT_ACTS[act], _dev(row_scale, "row_scale", torch.float32), _stream())
    y = torch.empty((pairs, width), dtype=torch.float32, device=x.device)
    _lib.call("pylon_grouped_down", _dev(y, "y"), _dev(hidden, "hidden"), ff, down.data_ptr(), down.stride(0),
              _dev(offsets, "offsets"), pairs, n_experts, ff, width, _stream())
    out = torch.empty((tokens, width), dtype=torch.float32, device=x.device)
    _lib.call("pylon_expert_combine", _dev(out, "out"), _dev(y, "y"), _dev(place, "place"),
              _dev(weights, "weights", torch.float32), _dev(shared, "shared", torch.float32),
              _dev(shared_gate, "shared_gate", torch.float32), tokens, top, width,
              offsets[n_experts:].data_ptr(),  # where the identities' pairs begin
              0 if identity_weight is None else x.data_ptr(), 0 if identity_weight is None else x.stride(0),
              _dev(identity_weight, "identity_weight", torch.float32), _stream())
    return out


def probe_read(data: torch.Tensor, sink: torch.Tensor) -> None:
    """Read every byte of ``data`` once (a measurement aid: the device's read bandwidth)."""
    if not data.is_contiguous() or not data.is_cuda:
        raise KernelError("probe_read takes a contiguous tensor on the GPU")
    _lib.call("pylon_probe_read", data.data_ptr(), data.numel() * data.element_size(),
              _dev(sink, "sink", torch.int32), _stream())

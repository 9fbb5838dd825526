"""Grouped-query attention over the paged cache
(/root/reference/src/pylon/model/layers.py:81-138; cache side
/root/reference/src/pylon/kv/cache.py:457-476).

``[q; k; v] = Wqkv h`` in one product, per-head RMSNorm of q and k (if the spec asks),
position encoding of q and k, k and v stored at the tokens' cache slots, causal softmax
attention of every token over its request's keys, output projection.  A run that borrows
another run's cache projects q only and stores nothing.

The spec may ask instead for one norm over the whole q projection and one over the whole k
projection (``qk_norm_over="projection"``), for a rotation that pairs neighbouring elements (the
position part's ``interleaved``) over a part of the head, for values of another size than keys,
and for keys visible inside the query's chunk of positions only (``chunk``); these go through
:func:`ops.qkv_prepare_wide` and the same attention kernels, which take the mask as one integer.

Further options of the spec: a rotation whose frequencies are stretched for long contexts and
whose cosines and sines carry a factor (the position part's ``rot_scale``); scores capped by
``softcap * tanh(s / softcap)``; a learned sink per head in the softmax's denominator; values that
are the keys as projected (``values_from_keys``: no value projection); and an output gate
``sigmoid(W_g h)`` per head or per element on the heads' outputs, whose rows are the last of the
fused projection ``[q; k; v; g]``.  Capped scores and the learned sink run, for bfloat16 over pages
of a multiple of 32 tokens, on the matrix-core kernel that :class:`SinkAttention` uses (prompt tiles and
single tokens with their keys cut over workgroups; the values then lie transposed inside their pages),
and otherwise on the general kernel.
"""
from __future__ import annotations

import torch

import math

from ..config.specs import AttentionSpec, SinkAttentionSpec
from ..kernels import ops
from .base import KVRequirement, Part
from .registry import build_part, register_part


class Attention(Part):
    def __init__(self, spec: AttentionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError("The number of Q heads must be divisible by the number of KV heads.")
        per_head = (not spec.qk_norm or spec.qk_norm_over == "head") and not getattr(spec.position, "interleaved", False) \
            and spec.value_dim == spec.head_dim and not spec.values_from_keys and spec.output_gate is None \
            and getattr(spec.position, "scaling", None) is None
        if per_head and (spec.head_dim % 16 or not 16 <= spec.head_dim <= 512):
            raise ValueError(
                f"head_dim {spec.head_dim} is not supported: the attention kernels take "
                "multiples of 16 from 16 to 512"
            )
        if not 1 <= spec.head_dim <= 512:
            raise ValueError(f"head_dim {spec.head_dim} is not supported: 1 to 512")
        if spec.window is not None and spec.window < 1:
            raise ValueError("window must be positive (or None for full attention)")
        if spec.chunk is not None and (spec.chunk < 1 or spec.window is not None):
            raise ValueError("chunk must be positive, and a layer has a window or chunks, not both")
        if spec.qk_norm_over not in ("head", "projection"):
            raise ValueError(f"qk_norm_over must be 'head' or 'projection', got {spec.qk_norm_over!r}")
        if spec.value_dim < 1 or spec.value_dim > 512:
            raise ValueError(f"value heads of {spec.value_dim} elements are not supported: 1 to 512")
        if spec.output_gate not in (None, "head", "element"):
            raise ValueError(f"output_gate must be None, 'head' or 'element', got {spec.output_gate!r}")
        if spec.values_from_keys and spec.value_dim != spec.head_dim:
            raise ValueError("values that are the keys have the keys' size")
        if spec.softcap is not None and not spec.softcap > 0:
            raise ValueError("a soft cap of the scores is positive")
        self.spec = spec
        self.dtype = dtype
        q, kv = spec.q_size, spec.kv_size
        # rows of the fused projection: q, k, v (none when the values are the keys), the gate
        self.v_rows = 0 if spec.values_from_keys else spec.v_size
        self.gate_off = q + kv + self.v_rows
        self.add_param("qkv", (self.gate_off + spec.gate_size, spec.hidden_size), dtype, device)
        if spec.sink:
            self.add_param("sink", (spec.n_heads,), torch.float32, device, role="vector")
        self.add_param("out", (spec.hidden_size, spec.n_heads * spec.value_dim), dtype, device)
        if spec.qk_norm:
            over_heads = spec.qk_norm_over == "head"
            self.add_param("q_norm", (spec.head_dim if over_heads else q,), torch.float32, device, role="vector")
            self.add_param("k_norm", (spec.head_dim if over_heads else kv,), torch.float32, device, role="vector")
        self.position = self.add_child("position", build_part("position", spec.position, dtype=dtype, device=device))
        # what the per-head preparation kernels (and the decode kernel that prepares its own
        # operands) cover: norms head by head, halves rotated together, values as large as keys
        self.plain = ((not spec.qk_norm or spec.qk_norm_over == "head") and spec.value_dim == spec.head_dim
                      and not getattr(self.position, "interleaved", False) and not spec.values_from_keys
                      and spec.output_gate is None and getattr(self.position, "rot_scale", 1.0) == 1.0)
        # capped scores and a learned sink: the general attention kernel
        self.special = spec.softcap is not None or spec.sink

    def cache_requirement(self) -> KVRequirement:
        spec = self.spec
        return KVRequirement(spec.n_kv_heads, spec.head_dim, spec.window,
                             v_head_dim=None if spec.value_dim == spec.head_dim else spec.value_dim, chunk=spec.chunk)

    def _span(self, ctx) -> int:
        """The most keys a token of this step attends to."""
        span = self.spec.window if self.spec.window is not None else self.spec.chunk
        return ctx.max_len if span is None else min(ctx.max_len, span)

    def decode_signature(self, rows: int, bound: int) -> tuple:
        """Of a bound on the lengths, a decode-only step's launches take only how the keys of
        a request are shared between workgroups and waves."""
        limit = self.spec.window if self.spec.window is not None else self.spec.chunk
        span = bound if limit is None else min(bound, limit)
        if self.special:
            if self.dtype != torch.bfloat16:
                return ("attention", "general")
            return ("attention", "sink", ops.sink_cuts(rows, self.spec.n_heads, self.spec.n_kv_heads, span))
        return ("attention",) + tuple(ops.decode_launch(rows, self.spec.n_kv_heads, span))

    def _sink_kernel(self, page_size: int) -> bool:
        """Whether capped scores and the sink run on the matrix cores (the values then lie transposed
        inside their pages: a property of the model's type, the heads' sizes and the page's, so every
        step of a runner stores and reads them one way)."""
        spec = self.spec
        return self.special and ops.attention_sink_ok(self.dtype, head_dim=spec.head_dim, v_dim=spec.value_dim,
                                                      page_size=page_size, bucket_len=0)

    def forward(self, h: torch.Tensor, ctx, cache, stores: bool) -> torch.Tensor:
        spec = self.spec
        tokens = h.shape[0]
        weight = self.params["qkv"]
        if not stores and spec.output_gate is None:
            weight = weight[: spec.q_size]
        rotary = self.position.rotary()
        mask = dict(window=spec.window, chunk=spec.chunk)
        if self.plain and not self.special and spec.chunk is None and ctx.decode_only and cache.k is not None and ops.decode_fused_ok(
                self.dtype, cache.k, tokens=tokens, n_heads=spec.n_heads, head_dim=spec.head_dim,
                rot_dim=rotary[1] if rotary else 0):
            # one launch adds the projection's partial sums if it comes as such, norms and
            # rotates q and k, stores k and v, and attends
            qkv = ops.linear_summed_later(h, weight, out_dtype=self.dtype)
            cuts, splits = ops.decode_launch(tokens, spec.n_kv_heads, self._span(ctx))
            context = ops.attention_decode_fused(
                qkv, cache.k, cache.v, cache.block_table, None, ctx.positions,
                n_heads=spec.n_heads, q_weight=self.params.get("q_norm"), k_weight=self.params.get("k_norm"),
                eps=spec.qk_norm_eps, inv_freq=rotary[0] if rotary else None,
                slot_map=cache.slot_map if stores else None,
                page_size=cache.page_size, window=spec.window, scale=spec.scale, n_splits=splits, n_cuts=cuts,
            )
            return ops.linear_for_residual(context.view(tokens, spec.q_size), self.params["out"],
                                           out_dtype=self.dtype)
        qkv = ops.linear(h, weight, out_dtype=self.dtype)
        q = torch.empty((tokens, spec.n_heads, spec.head_dim), dtype=self.dtype, device=h.device)
        on_cores = self._sink_kernel(cache.page_size) if cache.k is not None else False
        v_cache = cache.v
        if on_cores:
            v_cache = cache.v.view(cache.v.shape[0], spec.n_kv_heads, spec.value_dim, cache.page_size)
        if self.plain and not on_cores:
            ops.qkv_prepare(
                qkv, q, cache.k, cache.v,
                n_heads=spec.n_heads, n_kv_heads=spec.n_kv_heads, head_dim=spec.head_dim,
                q_weight=self.params.get("q_norm"), k_weight=self.params.get("k_norm"),
                eps=spec.qk_norm_eps,
                inv_freq=rotary[0] if rotary else None, rot_dim=rotary[1] if rotary else 0,
                positions=ctx.positions, slot_map=cache.slot_map, store_kv=stores,
            )
        else:
            # norms over whole projections, neighbours rotated together, values of another size
            ops.qkv_prepare_wide(
                qkv, q, cache.k, v_cache,
                n_heads=spec.n_heads, n_kv_heads=spec.n_kv_heads, head_dim=spec.head_dim, v_dim=spec.value_dim,
                q_weight=self.params.get("q_norm"), k_weight=self.params.get("k_norm"), eps=spec.qk_norm_eps,
                inv_freq=rotary[0] if rotary else None, rot_dim=rotary[1] if rotary else 0,
                interleaved=getattr(self.position, "interleaved", False),
                positions=ctx.positions, slot_map=cache.slot_map, store_kv=stores,
                per_head=spec.qk_norm and spec.qk_norm_over == "head",
                rot_scale=getattr(self.position, "rot_scale", 1.0), values_from_keys=spec.values_from_keys,
                v_transposed=on_cores,
            )
        # the matrix-core kernels take values as large as keys, plain scores and no sink
        same_size = spec.value_dim == spec.head_dim and not self.special
        if on_cores:
            tiles = None if ctx.decode_only else ctx.token_tiles(ops.SINK_TILE)
            cuts = ops.sink_cuts(tokens, spec.n_heads, spec.n_kv_heads, self._span(ctx)) if ctx.decode_only else 1
            context = ops.attention_sink(q, cache.k, v_cache, cache.block_table, tiles, ctx.positions,
                                         page_size=cache.page_size, scale=spec.scale, bias=None, sink=spec.sink,
                                         cuts=cuts, softcap=spec.softcap, sink_logit=self.params.get("sink"), **mask)
        elif same_size and ctx.decode_only and ops.decode_attention_ok(q, cache.k):
            cuts, splits = ops.decode_launch(tokens, spec.n_kv_heads, self._span(ctx))
            # in a decode-only step token t is row t
            context = ops.attention_decode(
                q, cache.k, cache.v, cache.block_table, None, ctx.positions,
                page_size=cache.page_size, scale=spec.scale, n_splits=splits, n_cuts=cuts, **mask,
            )
        elif same_size and ops.prefill_attention_ok(q, cache.k, cache.block_table):
            group = spec.n_heads // spec.n_kv_heads
            rows = ops.prefill_rows(tokens, spec.n_heads, group)
            context = torch.empty_like(q)
            # Decoding requests at the head of a mixed step go to the decode kernel (a
            # single query row would walk a long context alone in a prefill workgroup).
            singles = ctx.leading_singles
            if not (0 < singles <= ops.DECODE_MAX_TOKENS and ops.decode_attention_ok(q[:singles], cache.k)):
                singles = 0
            if singles:
                span = int(ctx.starts[:singles].max()) + 1
                if spec.window is not None or spec.chunk is not None:
                    span = min(span, spec.window if spec.window is not None else spec.chunk)
                cuts, splits = ops.decode_launch(singles, spec.n_kv_heads, span)
                ops.attention_decode(
                    q[:singles], cache.k, cache.v, cache.block_table, None, ctx.positions[:singles],
                    page_size=cache.page_size, scale=spec.scale, n_splits=splits,
                    n_cuts=cuts, out=context[:singles], **mask,
                )
            if singles < ctx.rows:
                tiles = ctx.token_tiles(rows // group, skip_rows=singles, fold=ops.prefill_fold(spec.n_kv_heads))
                ops.attention_prefill(
                    q, cache.k, cache.v, cache.block_table, tiles,
                    page_size=cache.page_size, scale=spec.scale, rows=rows, out=context, **mask,
                )
        else:
            context = ops.paged_attention(
                q, cache.k, cache.v, cache.block_table, ctx.tok_row, ctx.positions,
                page_size=cache.page_size, scale=spec.scale, softcap=spec.softcap,
                sink_logit=self.params.get("sink"), **mask,
            )
        context = context.view(tokens, spec.n_heads * spec.value_dim)
        if spec.output_gate is not None:
            ops.sigmoid_gate_(context, qkv[:, self.gate_off: self.gate_off + spec.gate_size],
                              per=spec.value_dim if spec.output_gate == "head" else 1)
        return ops.linear_for_residual(context, self.params["out"], out_dtype=self.dtype)


def distance_buckets(rows: int, far: float) -> list:
    """Row of a bias table of ``rows`` rows for every distance from 0 up to the first one that
    is at least ``far``: distances below ``rows // 2`` have a row each; from there on
    ``half + floor(log(n / half) / log(far / half) * (rows - half))``, capped at the last row,
    which every distance of at least ``far`` reaches.  Computed once, in double precision."""
    half = rows // 2
    if rows < 2 or not far > half:
        raise ValueError(f"a bias table of {rows} rows cannot spread its second half up to distance {far}")
    out = []
    for n in range(int(math.ceil(far)) + 1):
        if n < half:
            out.append(n)
        else:
            out.append(min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half)))))
    return out


class SinkAttention(Part):
    """Grouped-query attention over the paged cache with a learned bias by distance in place
    of a rotation, a sink in the softmax's denominator, and values of another size than keys.
    ``[q; k; v] = W h`` in one product; k and v go to the tokens' cache slots as they are, the
    values transposed inside their page (slot in page fastest), which is how the matrix-core
    kernel reads them; scores, bias and softmax are float32.  bfloat16 steps over pages of a
    multiple of 32 tokens run on the matrix cores (prompt portions as tiles of up to 32 tokens,
    a step of single tokens as one tile a token); everything else on the general kernel.

    The spec may ask instead for a bias that grows with the logarithm of the distance and is taken
    off the score, ``a_h * log(1 + b_h * (i - j))`` with two learned numbers per head
    (``bias_form="log"``; while a window or chunks bound the distances it reaches the matrix-core
    kernel as the same table by distance, computed once in float32); for keys visible inside the
    query's chunk of positions or a window only; for biases of the q, k and v projections (added to
    the product's float32 sums, rounded once, in the kernel that stores k and v); and for a layer
    that only ever runs on another run's keys and values (``own_kv`` False: q projection alone)."""

    def __init__(self, spec: SinkAttentionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError("The number of Q heads must be divisible by the number of KV heads.")
        if not 1 <= spec.head_dim <= 512 or not 1 <= spec.v_head_dim <= 512:
            raise ValueError(f"heads of {spec.head_dim} key and {spec.v_head_dim} value elements are not supported: "
                             "both take 1 to 512")
        if spec.window is not None and spec.window < 1:
            raise ValueError("window must be positive (or None for full attention)")
        if spec.chunk is not None and (spec.chunk < 1 or spec.window is not None):
            raise ValueError("chunk must be positive, and a layer has a window or chunks, not both")
        if spec.bias_form not in ("table", "log"):
            raise ValueError(f"bias_form must be 'table' or 'log', got {spec.bias_form!r}")
        self.spec = spec
        self.dtype = dtype
        self.q_size = spec.n_heads * spec.head_dim
        self.k_size = spec.n_kv_heads * spec.head_dim
        self.v_size = spec.n_kv_heads * spec.v_head_dim
        rows = self.q_size + (self.k_size + self.v_size if spec.own_kv else 0)
        self.add_param("qkv", (rows, spec.hidden_size), dtype, device)
        if spec.qkv_bias:
            self.add_param("qkv_bias", (rows,), torch.float32, device, role="vector")
        self.add_param("out", (spec.hidden_size, spec.n_heads * spec.v_head_dim), dtype, device)
        self.span = spec.window if spec.window is not None else spec.chunk  # the most keys a token sees (None: all)
        if spec.bias_form == "table":
            self.add_param("rel", (spec.bias_rows, spec.n_heads), torch.float32, device, role="vector")
            self.bucket = torch.tensor(distance_buckets(spec.bias_rows, spec.bias_far), dtype=torch.int32).to(device)
            self.bias_len = self.bucket.numel()
        else:
            # per head the factor a, then per head the slope b
            self.add_param("log_bias", (2 * spec.n_heads,), torch.float32, device, role="vector")
            self.bucket = None
            # as a table by distance it has one entry per distance a token can look back over
            self.bias_len = self.span if self.span is not None else ops.SINK_MAX_BIAS + 1
        self._bias = None  # (version of the parameter, the table by distance)

    def bias_by_distance(self) -> torch.Tensor:
        """The bias of every distance, float32 [heads, distances]: ``rel`` looked up, or ``-a log(1 + b
        d)`` evaluated, once; made anew when the parameter has been written since (a load, random
        weights drawn in place)."""
        source = self.params["rel"] if self.spec.bias_form == "table" else self.params["log_bias"]
        key = (source.data_ptr(), source._version)
        if self._bias is None or self._bias[0] != key:
            if self.spec.bias_form == "table":
                table = ops.bias_by_distance(source, self.bucket)
            else:
                a, b = source.view(2, self.spec.n_heads, 1)
                distance = torch.arange(self.bias_len, dtype=torch.float32, device=source.device)
                table = (-a * torch.log(1.0 + b * distance)).contiguous()
            self._bias = (key, table)
        return self._bias[1]

    def cache_requirement(self) -> KVRequirement:
        spec = self.spec
        if not spec.cache_bounded:
            return KVRequirement(spec.n_kv_heads, spec.head_dim, None, v_head_dim=spec.v_head_dim)
        return KVRequirement(spec.n_kv_heads, spec.head_dim, spec.window, v_head_dim=spec.v_head_dim, chunk=spec.chunk)

    def _matrix_cores(self, page_size: int) -> bool:
        spec = self.spec
        return ops.attention_sink_ok(self.dtype, head_dim=spec.head_dim, v_dim=spec.v_head_dim, page_size=page_size,
                                     bucket_len=self.bias_len)

    def decode_signature(self, rows: int, bound: int) -> tuple:
        """Of a bound on the lengths a step of single tokens takes only over how many workgroups
        a request's keys are cut."""
        if self.dtype != torch.bfloat16:
            return ("sink_attention",)
        span = bound if self.span is None else min(bound, self.span)
        return ("sink_attention", ops.sink_cuts(rows, self.spec.n_heads, self.spec.n_kv_heads, span))

    def forward(self, h: torch.Tensor, ctx, cache, stores: bool) -> torch.Tensor:
        spec = self.spec
        tokens = h.shape[0]
        if stores and not spec.own_kv:
            raise ValueError("a layer without k and v projections can only run on another run's keys and values")
        weight = self.params["qkv"] if stores else self.params["qkv"][: self.q_size]
        pages, page_size = cache.v.shape[0], cache.page_size
        v_cache = cache.v.view(pages, spec.n_kv_heads, spec.v_head_dim, page_size)
        if spec.qkv_bias:
            # the biases join the product's float32 sums; q, k and v are rounded once
            sums = ops.linear(h, weight, out_dtype=torch.float32)
            qkv = ops.qkv_bias_store(sums, self.params["qkv_bias"], cache.k, v_cache, cache.slot_map,
                                     q_size=self.q_size, k_size=self.k_size, v_size=self.v_size, out_dtype=self.dtype,
                                     store=stores, v_transposed=True)
        else:
            qkv = ops.linear(h, weight, out_dtype=self.dtype)
            if stores:
                ops.kv_store(qkv, cache.k, v_cache, cache.slot_map, k_off=self.q_size,
                             v_off=self.q_size + self.k_size, v_transposed=True)
        q = qkv.as_strided((tokens, spec.n_heads, spec.head_dim), (qkv.stride(0), spec.head_dim, 1))
        mask = dict(window=spec.window, chunk=spec.chunk)
        if self._matrix_cores(page_size) and qkv.stride(0) % 8 == 0:
            # tiles heaviest first (turning every second run of the order round, as the plain prefill
            # kernel's caller does, loses here: 227 -> 270 us a layer at 2,048 tokens with four waves a
            # workgroup, 5.81 -> 5.92 ms for eight layers with eight; the heaviest tile should start first)
            tiles = None if ctx.decode_only else ctx.token_tiles(ops.SINK_TILE)
            # a prompt portion's tiles keep their keys whole: cut in two or four, with the merge behind,
            # a 2,048-token prompt of eight layers took 6.18 and 6.58 ms against 5.82
            span = ctx.max_len if self.span is None else min(ctx.max_len, self.span)
            cuts = ops.sink_cuts(tokens, spec.n_heads, spec.n_kv_heads, span) if ctx.decode_only else 1
            context = ops.attention_sink(q, cache.k, v_cache, cache.block_table, tiles, ctx.positions,
                                         page_size=page_size, scale=spec.scale, bias=self.bias_by_distance(),
                                         sink=spec.sink, cuts=cuts, **mask)
        elif spec.bias_form == "table":
            context = ops.paged_attention(
                q, cache.k, v_cache, cache.block_table, ctx.tok_row, ctx.positions, page_size=page_size,
                scale=spec.scale, rel=self.params["rel"], bucket=self.bucket, sink=spec.sink,
                v_transposed=True, **mask)
        else:
            context = ops.paged_attention(
                q, cache.k, v_cache, cache.block_table, ctx.tok_row, ctx.positions, page_size=page_size,
                scale=spec.scale, log_bias=self.params["log_bias"].view(2, spec.n_heads), sink=spec.sink,
                v_transposed=True, **mask)
        return ops.linear_for_residual(context.view(tokens, spec.n_heads * spec.v_head_dim), self.params["out"],
                                       out_dtype=self.dtype)


register_part("mixer", "attention", Attention, replace=True)
register_part("mixer", "sink_attention", SinkAttention, replace=True)

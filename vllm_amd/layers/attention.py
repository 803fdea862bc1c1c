"""Attention layer: writes new K/V into the paged cache, then runs the
unified varlen attention op (prefill + decode in one call).

Role of the reference's Attention layer (layers/attention/attention.py:218)
with a single MI355X backend family instead of a backend registry.
"""

from __future__ import annotations


import torch
import torch.nn as nn

from vllm_amd import ops
from vllm_amd.worker.forward_context import get_forward_context


class Attention(nn.Module):
    def __init__(
        self,
        num_heads: int,
        head_dim: int,
        scale: float,
        num_kv_heads: int,
        layer_idx: int,
        sliding_window: int = 0,
        kv_group: str = "full",
    ):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.layer_idx = layer_idx
        self.sliding_window = sliding_window
        # "window": this layer reads/writes through the window group's
        # block table when the model has mixed sliding+global layers.
        self.kv_group = kv_group

    def forward(
        self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor
    ) -> torch.Tensor:
        """q: [T, Hq, D] or [T, Hq*D]; k/v likewise -> [T, Hq*D].

        Inputs may be strided head-slices of the fused QKV projection —
        the HIP kernels take row strides, so no contiguity copies here.
        """
        ctx = get_forward_context()
        meta = ctx.attn_metadata
        T = q.shape[0]
        if q.dim() == 2:
            q = q.view(T, self.num_heads, self.head_dim)
        if k.dim() == 2:
            k = k.view(T, self.num_kv_heads, self.head_dim)
        if v.dim() == 2:
            v = v.view(T, self.num_kv_heads, self.head_dim)

        if not ctx.kv_caches:
            # Memory-profiling run: no cache allocated; compute attention
            # over just the new tokens (worst-case activation footprint is
            # what matters, not values).
            return self._profile_attention(q, k, v, meta).reshape(T, -1)

        kv_cache = ctx.kv_caches[self.layer_idx]
        use_w = (self.kv_group == "window"
                 and meta.block_table_w is not None)
        slot_mapping = meta.slot_mapping_w if use_w else meta.slot_mapping
        block_table = meta.block_table_w if use_w else meta.block_table
        ops.reshape_and_cache(k, v, kv_cache, slot_mapping)
        out = ops.attention_unified(
            q,
            kv_cache,
            block_table,
            meta.query_start_loc,
            meta.seq_lens,
            self.scale,
            num_decodes=meta.num_decodes,
            sliding_window=self.sliding_window,
            max_seq_len=meta.max_seq_len,
            max_query_len=meta.max_query_len,
        )
        return out.reshape(T, -1)

    def _profile_attention(self, q, k, v, meta) -> torch.Tensor:
        """Cache-less varlen attention for the memory-profiling dummy run."""
        group = self.num_heads // self.num_kv_heads
        kk = k.repeat_interleave(group, dim=1)
        vv = v.repeat_interleave(group, dim=1)
        out = torch.empty_like(q)
        qs = meta.query_start_loc.tolist()
        for i in range(meta.num_reqs):
            s, e = qs[i], qs[i + 1]
            qi = q[s:e].transpose(0, 1).float()
            ki = kk[s:e].transpose(0, 1).float()
            vi = vv[s:e].transpose(0, 1).float()
            o = torch.nn.functional.scaled_dot_product_attention(
                qi, ki, vi, is_causal=True, scale=self.scale
            )
            out[s:e] = o.transpose(0, 1).to(out.dtype)
        return out


class PooledWindowAttention(nn.Module):
    """Sliding-window attention whose far context is kept as pooled
    blocks: position i attends the `window` most recent tokens and, for
    every block of `pool` consecutive tokens that lies wholly before
    that window, ONE key/value — the block's mean key and mean value.
    Window tokens and pooled blocks share one softmax. Positions do not
    enter the scores. Key and value head widths may differ.

    Cache per layer (allocated by the runner, paged by the same block
    table as every other model): k [blocks, G, block_size, D],
    v [blocks, G, block_size, Dv], and fp32 pooled areas
    [blocks, G, ceil(block_size / pool), D|Dv]; a pooled block is stored
    with the page that holds its last position, so it lives and dies
    with that page. Each step writes the new K/V, finalizes the pooled
    blocks the step completed (means of the keys as cached), then runs
    the varlen attention op over decodes and prefill chunks together.

    An optional per-head output gate (logits [T, H]) is applied in the
    attention epilogue: out[t, h] *= sigmoid(gate[t, h])."""

    def __init__(self, num_heads: int, head_dim: int, v_head_dim: int,
                 scale: float, num_kv_heads: int, window: int, pool: int):
        super().__init__()
        assert num_heads % num_kv_heads == 0
        assert window >= 1 and pool >= 1
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.v_head_dim = v_head_dim
        self.scale = scale
        self.window = window
        self.pool = pool

    def forward(self, q, k, v, gate, cache_idx: int,
                qk_norm=None) -> torch.Tensor:
        """q [T, H, D], k [T, G, D], v [T, G, Dv], gate [T, H] or None
        (all may be strided slices of one fused projection) ->
        [T, H * Dv]. qk_norm = (q_weight [D], k_weight [D], eps) applies
        a per-head RMS norm to q and k inside the cache-write pass."""
        ctx = get_forward_context()
        meta = ctx.attn_metadata
        T = q.shape[0]
        if not ctx.kv_caches:
            return self._profile_attention(q, k, v, gate, meta)
        k_cache, v_cache, pool_k, pool_v = ctx.kv_caches[cache_idx]
        q_w, k_w, eps = qk_norm if qk_norm is not None else (None, None, 0.0)
        q = ops.norm_qk_cache_write(q, k, v, q_w, k_w, eps, k_cache,
                                    v_cache, meta.slot_mapping)
        ops.pool_update(k_cache, v_cache, pool_k, pool_v, meta.block_table,
                        meta.query_start_loc, meta.seq_lens, self.pool,
                        max_query_len=meta.max_query_len)
        out = ops.pooled_window_attention(
            q, k_cache, v_cache, pool_k, pool_v, meta.block_table,
            meta.query_start_loc, meta.seq_lens, self.scale, self.window,
            self.pool, gate=gate, num_decodes=meta.num_decodes,
            max_seq_len=meta.max_seq_len,
            max_query_len=meta.max_query_len)
        return out.reshape(T, -1)

    def _profile_attention(self, q, k, v, gate, meta) -> torch.Tensor:
        """Memory-profiling run (no cache): only the activation footprint
        matters, so attend each token to itself."""
        group = self.num_heads // self.num_kv_heads
        out = v.repeat_interleave(group, dim=1)
        if gate is not None:
            out = out * torch.sigmoid(gate.float()).unsqueeze(-1).to(
                out.dtype)
        return out.reshape(q.shape[0], -1)


class LatentAttention(nn.Module):
    """Attention whose keys and values are both read from one cached
    latent row per token, shared by all heads: cache row = [c (kv_rank)
    | kr (rot_dim)]. A head's unrotated key is W_uk c and its value
    W_uv c, so the layer never expands them: queries are carried into
    the latent space (q_abs = W_uk^T q_nope, done by the caller), scores
    are (q_abs . c + q_rot . kr) * scale, and the kernel returns the
    attention-weighted latent [T, H, kv_rank] for the caller to expand
    through W_uv. Causal over the whole context.

    `sink` (one fp32 number per head, optional) is added to the softmax
    denominator as exp(sink_h): it has no key and no value.

    The same fused pass that writes the cache normalises c (RMS norm
    with a weight), rotates kr and the rotated part of q (PairwiseRotary).
    A layer built with writes_cache=False only reads: it attends over
    the rows another layer wrote into the cache it is pointed at.

    Cache per owning layer (allocated by the runner, paged by the
    ordinary block table): [blocks, block_size, kv_rank + rot_dim]."""

    def __init__(self, num_heads: int, nope_dim: int, rot_dim: int,
                 kv_rank: int, scale: float, rotary, eps: float,
                 cache_idx: int, writes_cache: bool = True,
                 has_sink: bool = False):
        super().__init__()
        self.num_heads = num_heads
        self.nope_dim = nope_dim
        self.rot_dim = rot_dim
        self.kv_rank = kv_rank
        self.scale = scale
        self.rotary = rotary
        self.eps = eps
        self.cache_idx = cache_idx
        self.writes_cache = writes_cache
        self.sink = (nn.Parameter(torch.zeros(num_heads,
                                              dtype=torch.float32),
                                  requires_grad=False)
                     if has_sink else None)

    def prepare(self, q, dkv, norm_w, positions):
        """Rotate q's rotated part in place; norm/rotate dkv and write
        it to the cache (when this layer owns one)."""
        ctx = get_forward_context()
        meta = ctx.attn_metadata
        cache = slots = None
        if ctx.kv_caches and self.writes_cache:
            cache = ctx.kv_caches[self.cache_idx]
            slots = meta.slot_mapping
        else:
            dkv = None
        ops.latent_rope_cache_write(
            q, dkv, norm_w, self.eps, positions, self.rotary.inv_freq,
            self.nope_dim, self.kv_rank, cache, slots)

    def forward(self, q_abs, q_rot) -> torch.Tensor:
        """q_abs [T, H, kv_rank], q_rot [T, H, rot_dim] (may be a strided
        view) -> [T, H, kv_rank]."""
        ctx = get_forward_context()
        meta = ctx.attn_metadata
        if not ctx.kv_caches:
            # Memory-profiling run: only the activation footprint counts.
            return torch.zeros_like(q_abs)
        return ops.latent_attention(
            q_abs, q_rot, ctx.kv_caches[self.cache_idx], meta.block_table,
            meta.query_start_loc, meta.seq_lens, self.scale,
            sink=self.sink, num_decodes=meta.num_decodes,
            max_seq_len=meta.max_seq_len,
            max_query_len=meta.max_query_len)

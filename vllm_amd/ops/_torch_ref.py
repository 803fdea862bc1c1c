"""Plain-PyTorch reference implementations of every custom op.

These are (a) the CPU execution path and (b) the numerics ground truth
for the HIP kernel tests (tests compare HIP output against these run in
fp32). Keep them simple and obviously correct.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    dtype = x.dtype
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps)
    return (out * weight.float()).to(dtype)


def fused_add_rms_norm(x, residual, weight, eps):
    new_residual = (x.float() + residual.float()).to(x.dtype)
    return rms_norm(new_residual, weight, eps), new_residual


def apply_rope(positions, q, k, cos_sin_cache, rotary_dim, is_neox=True):
    """In-place rotary embedding.

    positions: [T] int64; q: [T, Hq*D]; k: [T, Hkv*D];
    cos_sin_cache: [max_pos, rotary_dim] = concat(cos, sin) halves.
    """
    num_tokens = positions.shape[0]
    cos_sin = cos_sin_cache[positions]  # [T, rotary_dim]
    cos, sin = cos_sin.chunk(2, dim=-1)  # [T, rotary_dim/2] each

    def rotate(t: torch.Tensor) -> torch.Tensor:
        # t: [T, H, D]; rotate the first rotary_dim of D.
        rot = t[..., :rotary_dim].float()
        if is_neox:
            x1, x2 = rot.chunk(2, dim=-1)
            c = cos.unsqueeze(1).float()
            s = sin.unsqueeze(1).float()
            o1 = x1 * c - x2 * s
            o2 = x2 * c + x1 * s
            rotated = torch.cat([o1, o2], dim=-1)
        else:  # GPT-J interleaved
            x1 = rot[..., ::2]
            x2 = rot[..., 1::2]
            c = cos.unsqueeze(1).float()
            s = sin.unsqueeze(1).float()
            o1 = x1 * c - x2 * s
            o2 = x2 * c + x1 * s
            rotated = torch.stack([o1, o2], dim=-1).flatten(-2)
        t[..., :rotary_dim] = rotated.to(t.dtype)
        return t

    if q.dim() != 3 or k.dim() != 3:
        raise ValueError("apply_rope expects q/k as [T, H, D] views")
    rotate(q)
    rotate(k)
    return q, k


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    return F.silu(x[..., :d].float()).to(x.dtype) * x[..., d:]


def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.shape[-1] // 2
    return F.gelu(x[..., :d].float(), approximate="tanh").to(x.dtype) * x[..., d:]


def reshape_and_cache(key, value, kv_cache, slot_mapping):
    """key/value: [T, Hkv, D]; kv_cache: [2, num_blocks, Hkv, block_size, D]
    (head-major inside the block — each (block, head) tile is one contiguous
    chunk for the HIP kernels); slot_mapping: [T] int64
    (block_id * block_size + offset)."""
    block_size = kv_cache.shape[3]
    block_ids = slot_mapping // block_size
    offsets = slot_mapping % block_size
    kv_cache[0, block_ids, :, offsets] = key.to(kv_cache.dtype)
    kv_cache[1, block_ids, :, offsets] = value.to(kv_cache.dtype)


def _gather_kv(kv_cache, block_table_row, ctx_len):
    """Gather [ctx_len, Hkv, D] K and V for one request from paged cache."""
    block_size = kv_cache.shape[3]
    num_blocks_needed = (ctx_len + block_size - 1) // block_size
    blocks = block_table_row[:num_blocks_needed].long()
    k = kv_cache[0, blocks]  # [nb, Hkv, bs, D]
    v = kv_cache[1, blocks]
    k = k.transpose(1, 2).reshape(-1, k.shape[1], k.shape[3])[:ctx_len]
    v = v.transpose(1, 2).reshape(-1, v.shape[1], v.shape[3])[:ctx_len]
    return k, v


def attention_unified(
    q,
    kv_cache,
    block_table,
    query_start_loc,
    seq_lens,
    scale,
    num_decodes=0,
    sliding_window=0,
    max_seq_len=0,
    max_query_len=0,
):
    num_tokens, num_heads, head_dim = q.shape
    num_kv_heads = kv_cache.shape[2]
    group = num_heads // num_kv_heads
    head_dim_v = kv_cache.shape[4]
    out = q.new_empty(num_tokens, num_heads, head_dim_v)
    num_reqs = seq_lens.shape[0]
    qs = query_start_loc.tolist()
    for i in range(num_reqs):
        q_start, q_end = qs[i], qs[i + 1]
        ql = q_end - q_start
        ctx = int(seq_lens[i])
        qi = q[q_start:q_end].float()  # [ql, H, D]
        k, v = _gather_kv(kv_cache, block_table[i], ctx)
        k = k.float().repeat_interleave(group, dim=1)  # [ctx, H, D]
        v = v.float().repeat_interleave(group, dim=1)
        # scores: [H, ql, ctx]
        scores = torch.einsum("qhd,khd->hqk", qi, k) * scale
        # Causal mask: query j (global pos ctx-ql+j) sees keys <= its pos.
        kpos = torch.arange(ctx, device=q.device)
        qpos = ctx - ql + torch.arange(ql, device=q.device)
        mask = kpos.unsqueeze(0) > qpos.unsqueeze(1)  # [ql, ctx]
        if sliding_window > 0:
            mask |= kpos.unsqueeze(0) <= (qpos.unsqueeze(1) - sliding_window)
        scores.masked_fill_(mask.unsqueeze(0), float("-inf"))
        p = scores.softmax(dim=-1)
        o = torch.einsum("hqk,khd->qhd", p, v)
        out[q_start:q_end] = o.to(out.dtype)
    return out


def linear(x, weight, bias=None):
    return F.linear(x, weight, bias)


FP8_MAX = 448.0  # OCP e4m3fn max finite


def quant_fp8_dynamic(x):
    """Per-token (row) dynamic fp8 quantization.

    x: [M, K] -> (x_fp8 [M, K] float8_e4m3fn, scales [M] f32). Ground
    truth for the HIP kernel in csrc/quant_fp8.hip."""
    xf = x.float()
    amax = xf.abs().amax(dim=-1).clamp_min(1e-12)
    scales = amax / FP8_MAX
    q = (xf / scales.unsqueeze(1)).to(torch.float8_e4m3fn)
    return q, scales


def quantize_weight_fp8(w):
    """Per-output-channel fp8 weight quantization (done once at load).

    w: [N, K] -> (w_fp8 [N, K] float8_e4m3fn, scales [N] f32)."""
    wf = w.float()
    amax = wf.abs().amax(dim=-1).clamp_min(1e-12)
    scales = amax / FP8_MAX
    q = (wf / scales.unsqueeze(1)).to(torch.float8_e4m3fn)
    return q, scales


def linear_fp8(x, w_fp8, w_scale, bias=None):
    """W8A8 fp8 linear, CPU reference: quantize activations per-token
    exactly as the GPU path does, then compute in fp32 on dequantized
    values (same rounding points as fp8-GEMM + rs*cs rescale)."""
    shape = list(x.shape)
    x2 = x.reshape(-1, shape[-1])
    x_fp8, x_scale = quant_fp8_dynamic(x2)
    y = x_fp8.float() @ w_fp8.float().t()
    y = y * x_scale.unsqueeze(1) * w_scale.unsqueeze(0)
    if bias is not None:
        y = y + bias.float()
    shape[-1] = w_fp8.shape[0]
    return y.to(x.dtype).reshape(shape)


def topk_softmax(gating_logits, topk, renormalize=True):
    """gating_logits: [T, E] -> (topk_weights [T,k] f32, topk_ids [T,k] i32)."""
    probs = gating_logits.float().softmax(dim=-1)
    topk_weights, topk_ids = probs.topk(topk, dim=-1)
    if renormalize:
        topk_weights = topk_weights / topk_weights.sum(dim=-1, keepdim=True)
    return topk_weights, topk_ids.to(torch.int32)


def fused_moe(hidden, w13, w2, topk_weights, topk_ids, activation="silu"):
    """Reference MoE: loop over experts.

    hidden: [T, H]; w13: [E, 2I, H]; w2: [E, H, I];
    topk_weights/topk_ids: [T, k]. Returns [T, H]. activation "relu2"
    is not gated: w13 is the up projection alone, [E, I, H].
    """
    T, H = hidden.shape
    E = w13.shape[0]
    out = torch.zeros(T, H, dtype=torch.float32, device=hidden.device)
    act = {"silu": silu_and_mul, "gelu": gelu_and_mul,
           "relu2": relu2}[activation]
    flat_ids = topk_ids.long()
    for e in range(E):
        mask = flat_ids == e  # [T, k]
        if not mask.any():
            continue
        token_idx, k_idx = mask.nonzero(as_tuple=True)
        x = hidden[token_idx]
        h = act(x @ w13[e].t())
        y = h @ w2[e].t()
        w = topk_weights[token_idx, k_idx].unsqueeze(-1).float()
        out.index_add_(0, token_idx, y.float() * w)
    return out.to(hidden.dtype)


def concat_and_cache_mla(c_kv, k_pe, kv_cache, slot_mapping):
    """MLA cache write: c_kv [T, lora], k_pe [T, rope] ->
    kv_cache [num_blocks, block_size, lora+rope]."""
    block_size = kv_cache.shape[1]
    blk = slot_mapping // block_size
    off = slot_mapping % block_size
    lora = c_kv.shape[1]
    kv_cache[blk, off, :lora] = c_kv
    kv_cache[blk, off, lora:] = k_pe


def mla_attention(
    q_nope,       # [T, Hq, d_nope]  (already absorbed: d_nope == kv_lora)
    q_pe,         # [T, Hq, d_rope]
    kv_cache,     # [num_blocks, block_size, kv_lora + d_rope]
    block_table,  # [num_reqs, max_blocks] int32
    query_start_loc,  # [num_reqs+1]
    seq_lens,     # [num_reqs]
    scale,
):
    """Attention in the compressed (absorbed) MLA space: scores =
    q_nope . c_kv + q_pe . k_pe; output is in kv_lora space [T, Hq, lora]
    (caller applies W_UV). Causal over each request's own new tokens.

    Role of the reference's MLA backends (vllm/v1/attention/backends/mla/)
    in plain torch — the numerics ground truth for the HIP MLA kernel.
    """
    T, Hq, lora = q_nope.shape
    d_rope = q_pe.shape[2]
    block_size = kv_cache.shape[1]
    out = q_nope.new_empty(T, Hq, lora)
    qs = query_start_loc.tolist()
    num_reqs = seq_lens.shape[0]
    for i in range(num_reqs):
        s, e = qs[i], qs[i + 1]
        ql = e - s
        ctx = int(seq_lens[i])
        nb = (ctx + block_size - 1) // block_size
        blocks = block_table[i, :nb].long()
        kv = kv_cache[blocks].reshape(-1, lora + d_rope)[:ctx].float()
        c_kv, k_pe = kv[:, :lora], kv[:, lora:]
        qn = q_nope[s:e].float()  # [ql, Hq, lora]
        qp = q_pe[s:e].float()
        scores = (
            torch.einsum("qhl,kl->hqk", qn, c_kv)
            + torch.einsum("qhr,kr->hqk", qp, k_pe)
        ) * scale
        kpos = torch.arange(ctx, device=qn.device)
        qpos = ctx - ql + torch.arange(ql, device=qn.device)
        mask = kpos.unsqueeze(0) > qpos.unsqueeze(1)
        scores.masked_fill_(mask.unsqueeze(0), float("-inf"))
        p = scores.softmax(dim=-1)
        o = torch.einsum("hqk,kl->qhl", p, c_kv)
        out[s:e] = o.to(out.dtype)
    return out


def grouped_topk(
    gating, topk, renormalize=True, num_groups=0, topk_groups=0,
    scoring_func="softmax", e_score_bias=None, routed_scaling_factor=1.0,
):
    """DeepSeek-style routing: sigmoid/softmax scoring, optional
    group-limited expert selection (n_group/topk_group), optional
    per-expert score bias (role of fused_moe grouped_topk)."""
    T, E = gating.shape
    if scoring_func == "sigmoid":
        scores = gating.float().sigmoid()
    else:
        scores = gating.float().softmax(dim=-1)
    select = scores if e_score_bias is None else scores + e_score_bias
    if num_groups > 0 and topk_groups > 0:
        g = select.view(T, num_groups, E // num_groups)
        # Group score: sum of top-2 experts inside each group.
        group_score = g.topk(min(2, g.shape[-1]), dim=-1).values.sum(-1)
        keep = group_score.topk(topk_groups, dim=-1).indices
        mask = torch.zeros(T, num_groups, dtype=torch.bool,
                           device=gating.device)
        mask.scatter_(1, keep, True)
        select = select.masked_fill(
            ~mask.unsqueeze(-1).expand_as(g).reshape(T, E), float("-inf")
        )
    topk_ids = select.topk(topk, dim=-1).indices
    topk_weights = scores.gather(1, topk_ids)
    if renormalize:
        topk_weights = topk_weights / topk_weights.sum(-1, keepdim=True)
    topk_weights = topk_weights * routed_scaling_factor
    return topk_weights, topk_ids.to(torch.int32)


# ---------------------------------------------------------------------
# fp32 residual stream, token shift, scalar-gain RMS norm, and the
# sliding-window attention with mean-pooled far blocks.

def scalar_rms_norm(x, gain, eps, out_dtype=None):
    """x / sqrt(mean(x^2) + eps) * gain with ONE gain for the whole row
    (gain: 0-dim tensor). Math in fp32; result in out_dtype (fp32 when
    None)."""
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf / torch.sqrt(var + eps) * gain.float()
    return out.to(out_dtype or torch.float32)


def add_scaled_scalar_norm(residual, y, gain, eps, mult, out_dtype=None):
    """residual += mult * scalar_rms_norm(y, gain), in place on the fp32
    residual stream. Returns the updated residual, as a copy in
    out_dtype when one is asked for (input of the next GEMM)."""
    residual.add_(scalar_rms_norm(y, gain, eps), alpha=mult)
    if out_dtype is None or out_dtype == residual.dtype:
        return residual
    return residual.to(out_dtype)


def token_shift(x, shift, state, state_rows, query_start_loc, out_dtype):
    """h[t] + (h[t-1] - h[t]) * shift per sequence; the token before a
    chunk's first one comes from state[state_rows[r]] (zeros for a fresh
    sequence), and the chunk's last h is stored back there. x: [T, W]
    fp32; state: [rows, W] fp32 or None (no carry: zeros)."""
    T = x.shape[0]
    prev = torch.empty_like(x)
    prev[1:] = x[:-1]
    qs = query_start_loc.tolist()
    for r in range(len(qs) - 1):
        s, e = qs[r], qs[r + 1]
        if s == e:
            continue
        if state is not None:
            row = int(state_rows[r])
            prev[s] = state[row]
            state[row] = x[e - 1]
        else:
            prev[s] = 0
    return (x + (prev - x) * shift.float()).to(out_dtype)


def split_cache_write(key, value, k_cache, v_cache, slot_mapping):
    """key [T, G, D] -> k_cache [blocks, G, block_size, D]; value
    [T, G, Dv] -> v_cache [blocks, G, block_size, Dv] (key and value
    widths may differ). Slots < 0 are skipped."""
    block_size = k_cache.shape[2]
    keep = slot_mapping >= 0
    slots = slot_mapping[keep]
    blk = slots // block_size
    off = slots % block_size
    k_cache[blk, :, off] = key[keep].to(k_cache.dtype)
    v_cache[blk, :, off] = value[keep].to(v_cache.dtype)


def norm_qk_cache_write(q, k, v, q_w, k_w, eps, k_cache, v_cache,
                        slot_mapping):
    """Per-head RMS norm of q and k (weights [D] shared by all heads;
    None = no norm), then the paged K/V write. Returns the normed q
    [T, H, D], contiguous."""
    if q_w is not None:
        q = rms_norm(q.reshape(-1, q.shape[-1]), q_w, eps).view(q.shape)
        k = rms_norm(k.reshape(-1, k.shape[-1]), k_w, eps).view(k.shape)
    split_cache_write(k, v, k_cache, v_cache, slot_mapping)
    return q.contiguous()


def _pool_slot(b, pool, block_size):
    """Pooled block b (positions b*pool .. b*pool+pool-1) is stored with
    the page that holds its LAST position; pages are block_size tokens.
    Returns (logical page, slot inside that page's pooled area)."""
    page = (b * pool + pool - 1) // block_size
    return page, b - (page * block_size) // pool


def pool_slots_per_page(pool, block_size):
    return -(-block_size // pool)


def pool_update(k_cache, v_cache, pool_k, pool_v, block_table,
                query_start_loc, seq_lens, pool):
    """Mean key/value of every pooled block that this step completed
    (its last position was written this step), read back from the cache
    as stored. pool_k/pool_v: [blocks, G, slots_per_page, D] fp32."""
    bs = k_cache.shape[2]
    qs = query_start_loc.tolist()
    sl = seq_lens.tolist()
    for r in range(len(sl)):
        n = qs[r + 1] - qs[r]
        end = sl[r]
        start = end - n
        # blocks whose last position b*pool + pool - 1 is in [start, end)
        for b in range(start // pool, end // pool):
            pos = torch.arange(b * pool, b * pool + pool,
                               device=k_cache.device)
            blk = block_table[r, pos // bs].long()
            off = pos % bs
            km = k_cache[blk, :, off].float().mean(0)   # [G, D]
            vm = v_cache[blk, :, off].float().mean(0)
            page, slot = _pool_slot(b, pool, bs)
            pb = int(block_table[r, page])
            pool_k[pb, :, slot] = km
            pool_v[pb, :, slot] = vm


def pooled_window_attention(q, k_cache, v_cache, pool_k, pool_v,
                            block_table, query_start_loc, seq_lens, scale,
                            window, pool, gate=None, num_decodes=0,
                            max_seq_len=0, max_query_len=0):
    """Position i attends the tokens j with 0 <= i - j < window plus one
    pooled (mean) key/value per block of `pool` tokens that lies wholly
    before the window (b*pool + pool - 1 <= i - window); one softmax
    over both. gate: [T, H] logits — head outputs are multiplied by
    sigmoid(gate). q: [T, H, D] -> [T, H, Dv]."""
    T, H, D = q.shape
    G = k_cache.shape[1]
    Dv = v_cache.shape[3]
    bs = k_cache.shape[2]
    group = H // G
    out = torch.empty(T, H, Dv, dtype=q.dtype, device=q.device)
    qs = query_start_loc.tolist()
    sl = seq_lens.tolist()
    for r in range(len(sl)):
        s, e = qs[r], qs[r + 1]
        n = e - s
        if n == 0:
            continue
        L = sl[r]
        pos = torch.arange(L, device=q.device)
        blk = block_table[r, pos // bs].long()
        k_all = k_cache[blk, :, pos % bs].float()   # [L, G, D]
        v_all = v_cache[blk, :, pos % bs].float()
        nb_max = max(0, (L - 1 - window + 1) // pool)
        if nb_max:
            pk = torch.stack([
                pool_k[int(block_table[r, _pool_slot(b, pool, bs)[0]]), :,
                       _pool_slot(b, pool, bs)[1]] for b in range(nb_max)])
            pv = torch.stack([
                pool_v[int(block_table[r, _pool_slot(b, pool, bs)[0]]), :,
                       _pool_slot(b, pool, bs)[1]] for b in range(nb_max)])
        for t in range(n):
            i = L - n + t
            lo = max(0, i - window + 1)
            nb = max(0, (i - window + 1) // pool)
            kk = k_all[lo:i + 1]
            vv = v_all[lo:i + 1]
            if nb:
                kk = torch.cat([pk[:nb].float(), kk])
                vv = torch.cat([pv[:nb].float(), vv])
            kk = kk.repeat_interleave(group, dim=1)   # [n, H, D]
            vv = vv.repeat_interleave(group, dim=1)
            sc = torch.einsum("hd,nhd->hn", q[s + t].float(), kk) * scale
            p = torch.softmax(sc, dim=-1)
            o = torch.einsum("hn,nhd->hd", p, vv)
            if gate is not None:
                o = o * torch.sigmoid(gate[s + t].float()).unsqueeze(-1)
            out[s + t] = o.to(out.dtype)
    return out


# ---------------------------------------------------------------------
# fp32 residual stream with weighted output norms, latent attention
# with a softmax sink over a shared latent cache, state-space-duality
# (Mamba-2) mixers, squared-relu experts.

def scaled_embedding(input_ids, table, scale):
    """fp32 rows table[id] * scale."""
    return table[input_ids].float() * scale


def rms_norm_cast(x, weight, eps, out_dtype):
    """x / sqrt(mean(x^2) + eps) * w in fp32, stored as out_dtype."""
    xf = x.float()
    inv = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * inv * weight.float()).to(out_dtype)


def add_rms_norm(residual, y, weight, eps, out_dtype=None):
    """residual (fp32, in place) += norm(y) * w. Returns the updated
    residual, as a copy in out_dtype when that is a 16-bit type."""
    yf = y.float()
    inv = torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps)
    residual.add_(yf * inv * weight.float())
    if out_dtype is None or out_dtype == torch.float32:
        return residual
    return residual.to(out_dtype)


def relu2(x):
    r = torch.relu(x)
    return r * r


def logit_softcap(logits, cap):
    return cap * torch.tanh(logits.float() / cap)


def softmax_topk_scaled(logits, topk, scale):
    """Softmax over all experts (fp32), the topk largest, each divided
    by their sum (+1e-20) and multiplied by scale."""
    probs = logits.float().softmax(dim=-1)
    w, ids = probs.topk(topk, dim=-1)
    w = w / (w.sum(dim=-1, keepdim=True) + 1e-20) * scale
    return w, ids.to(torch.int32)


def _rotate_pairs(v, positions, inv_freq):
    """v [T, ..., n] float; pairs (2i, 2i+1) for i < len(inv_freq) turn
    by positions * inv_freq[i]; the remaining coordinates pass."""
    n2 = inv_freq.shape[0] * 2
    if n2 == 0:
        return v
    ang = positions.float().unsqueeze(-1) * inv_freq.float()
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [n2 // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, w = v[..., 0:n2:2], v[..., 1:n2:2]
    out = v.clone()
    out[..., 0:n2:2] = u * c - w * s
    out[..., 1:n2:2] = w * c + u * s
    return out


def latent_rope_cache_write(q, dkv, norm_w, eps, positions, inv_freq,
                            nope_dim, kv_rank, cache, slot_mapping):
    """q [T, H, nope+rot] (modified in place): the last rot coordinates
    of every head are rotated. dkv [T, kv_rank+rot] or None: the first
    kv_rank coordinates are RMS-normed (weight norm_w), the rest
    rotated, and the row is written to cache [blocks, page, kv_rank+rot]
    at slot_mapping (negative slots are skipped)."""
    qr = q[..., nope_dim:]
    qr.copy_(_rotate_pairs(qr.float(), positions, inv_freq).to(q.dtype))
    if dkv is None:
        return
    d = dkv.float()
    c = d[:, :kv_rank]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) \
        * norm_w.float()
    kr = _rotate_pairs(d[:, kv_rank:], positions, inv_freq)
    row = torch.cat([c, kr], dim=-1).to(cache.dtype)
    ok = slot_mapping >= 0
    flat = cache.view(-1, cache.shape[-1])
    flat[slot_mapping[ok]] = row[ok]


def latent_attention(q_abs, q_rot, cache, block_table, query_start_loc,
                     seq_lens, scale, sink=None, num_decodes=0,
                     max_seq_len=0, max_query_len=0):
    """Causal attention of every head over ONE shared latent stream.
    q_abs [T, H, L] (queries already carried into the latent space),
    q_rot [T, H, R], cache [blocks, page, L+R]; score = (q_abs . c +
    q_rot . kr) * scale; value = c. sink [H] adds exp(sink_h) to the
    softmax denominator (no key, no value, not scaled). -> [T, H, L]."""
    T, H, L = q_abs.shape
    page = cache.shape[1]
    out = torch.zeros(T, H, L, dtype=q_abs.dtype, device=q_abs.device)
    qsl = query_start_loc.tolist()
    lens = seq_lens.tolist()
    for r in range(len(lens)):
        s, e = qsl[r], qsl[r + 1]
        n, ctx = e - s, lens[r]
        if n == 0 or ctx == 0:
            continue
        nb = -(-ctx // page)
        rows = cache[block_table[r, :nb].long()].reshape(
            nb * page, -1)[:ctx].float()
        c, kr = rows[:, :L], rows[:, L:]
        sc = (torch.einsum("nhl,kl->hnk", q_abs[s:e].float(), c)
              + torch.einsum("nhr,kr->hnk", q_rot[s:e].float(), kr)) * scale
        pos = torch.arange(ctx - n, ctx, device=sc.device)
        hide = torch.arange(ctx, device=sc.device)[None, :] > pos[:, None]
        sc = sc.masked_fill(hide[None], float("-inf"))
        if sink is not None:
            extra = sink.float().view(H, 1, 1).expand(H, n, 1)
            p = torch.cat([sc, extra], dim=-1).softmax(dim=-1)[..., :ctx]
        else:
            p = sc.softmax(dim=-1)
        out[s:e] = torch.einsum("hnk,kl->nhl", p, c).to(out.dtype)
    return out


def sigmoid_gate_mul(x, gate):
    """x [T, H, D] (any strides) * sigmoid(gate [T, H*D]) ->
    contiguous [T, H*D]."""
    xf = x.reshape(x.shape[0], -1).float()
    return (xf * torch.sigmoid(gate.float())).to(x.dtype).contiguous()


def causal_conv_silu(x, weight, bias, conv_state, state_rows,
                     query_start_loc, out_dtype=None):
    """Per-channel causal convolution + silu over a varlen batch.
    x [T, C]; weight [C, K] (last tap = current token); conv_state
    [rows, C, K-1] holds each request's last K-1 inputs (oldest first)
    and is advanced in place; None = zero history, nothing kept.
    Returns a contiguous [T, C] in out_dtype (default: x's)."""
    T, C = x.shape
    K = weight.shape[1]
    out = torch.empty(T, C, dtype=out_dtype or x.dtype, device=x.device)
    qsl = query_start_loc.tolist()
    wf, bf = weight.float(), bias.float()
    for r in range(len(qsl) - 1):
        s, e = qsl[r], qsl[r + 1]
        if s == e:
            continue
        if conv_state is not None:
            row = int(state_rows[r])
            hist = conv_state[row].float()
        else:
            hist = torch.zeros(C, K - 1, device=x.device)
        ext = torch.cat([hist, x[s:e].float().t()], dim=1)  # [C, K-1+n]
        if conv_state is not None and K > 1:
            conv_state[row] = ext[:, ext.shape[1] - (K - 1):].to(
                conv_state.dtype)
        win = ext.unfold(1, K, 1)                           # [C, n, K]
        y = (win * wf[:, None, :]).sum(-1) + bf[:, None]
        out[s:e] = (y * torch.sigmoid(y)).t().to(out.dtype)
    return out


def ssd_scan(xbc, heads, head_dim, groups, state, dt, dt_bias, a_log,
             d_skip, ssm_state, state_rows, query_start_loc):
    """State-space-duality recurrence per head over a varlen batch.
    xbc [T, heads*head_dim + 2*groups*state] = x | B | C; dt [T, heads]
    (raw); ssm_state [rows, heads, head_dim, state] fp32 advanced in
    place (None = zero start). Head h uses B/C group h // (heads/groups).
      dt' = softplus(dt + dt_bias);  S <- exp(-exp(a_log) dt') S
      + dt' x B^T;  y = S C + d_skip x.     -> y fp32 [T, heads, head_dim]"""
    T = xbc.shape[0]
    Hm, P, G, N = heads, head_dim, groups, state
    inner = Hm * P
    per = Hm // G
    xf = xbc[:, :inner].float().view(T, Hm, P)
    Bh = xbc[:, inner:inner + G * N].float().view(
        T, G, N).repeat_interleave(per, dim=1)                 # [T, Hm, N]
    Ch = xbc[:, inner + G * N:].float().view(
        T, G, N).repeat_interleave(per, dim=1)
    y = torch.empty(T, Hm, P, dtype=torch.float32, device=xbc.device)
    dtp = torch.nn.functional.softplus(dt.float() + dt_bias.float())
    decay = torch.exp(-torch.exp(a_log.float()) * dtp)        # [T, Hm]
    qsl = query_start_loc.tolist()
    for r in range(len(qsl) - 1):
        s, e = qsl[r], qsl[r + 1]
        if s == e:
            continue
        if ssm_state is not None:
            row = int(state_rows[r])
            S = ssm_state[row].clone()
        else:
            S = torch.zeros(Hm, P, N, device=xbc.device)
        for t in range(s, e):
            S = decay[t, :, None, None] * S + dtp[t, :, None, None] * (
                xf[t, :, :, None] * Bh[t, :, None, :])
            y[t] = (S * Ch[t, :, None, :]).sum(-1)
        if ssm_state is not None:
            ssm_state[row] = S
    return y + d_skip.float()[None, :, None] * xf


def gated_group_rms_norm(y, z, weight, eps, groups, out_dtype):
    """(y * silu(z)) normed in `groups` equal parts, each by its own
    root mean square, times weight. y fp32 [T, W], z [T, W]."""
    T, W = y.shape
    zf = z.float()
    g = y.float() * (zf * torch.sigmoid(zf))
    g = g.view(T, groups, W // groups)
    g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)
    return (g.reshape(T, W) * weight.float()).to(out_dtype)

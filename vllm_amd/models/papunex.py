"""Papunex: a decoder-only stack listed layer by layer in config.json
(sizes, constants and layer order all come from there).

    x = embed[token] * embedding_scale                    fp32 stream
    per layer:  x += norm1(mixer(x))
                x += norm2(ff(x))                         if it has one
    logits = softcap(head(norm_f(x)))

- Norms (RMS, weighted) sit on the sublayer's OUTPUT; sublayers read
  the residual stream itself, which stays fp32 in every compute dtype
  (layers/layernorm.py RMSNorm.add_into).
- Mixer "latent_attention" (layers/attention.py LatentAttention): one
  cached latent row [c | kr] per token serves every head. q | dkv |
  gate come out of ONE fused GEMM; the cache-write pass norms c and
  rotates kr and q's rotated part; queries are carried into the latent
  space through W_uk, the attention result is expanded through W_uv,
  multiplied by sigmoid(gate) and projected out. The softmax has a
  learned per-head sink. A layer with "kv_from": j has no key
  projection and reads the cache layer j wrote.
- Mixer "mamba2" (layers/mamba2.py Mamba2Mixer): state-space duality
  with per-request conv tail and fp32 state in runner rows.
- Feed-forward: dense squared-relu MLP, or routed squared-relu experts
  (layers/fused_moe.py SoftmaxTopKRouter + FusedMoE.run_experts) plus
  an optional shared expert scaled by a per-token sigmoid gate.

Tensor parallelism is not implemented for this family (tp must be 1).
"""

from __future__ import annotations

import torch
import torch.nn as nn

from vllm_amd import ops
from vllm_amd.config import ModelConfig
from vllm_amd.layers.attention import LatentAttention
from vllm_amd.layers.embedding import ParallelLMHead, VocabParallelEmbedding
from vllm_amd.layers.fused_moe import FusedMoE, SoftmaxTopKRouter
from vllm_amd.layers.layernorm import RMSNorm
from vllm_amd.layers.linear import ReplicatedLinear
from vllm_amd.layers.mamba2 import Mamba2Mixer
from vllm_amd.layers.rotary import PairwiseRotary
from vllm_amd.parallel.state import get_tp_world_size


def _round_up(n: int, m: int) -> int:
    return -(-n // m) * m


class PapunexLatentMixer(nn.Module):

    def __init__(self, width: int, mx: dict, eps: float, cache_idx: int,
                 dtype: torch.dtype):
        super().__init__()
        self.H = int(mx["heads"])
        self.D = int(mx["dim"])
        self.R = int(mx["rot_dim"])
        self.Dv = int(mx["vdim"])
        self.L = int(mx["kv_rank"])
        self.owns_kv = mx.get("kv_from") is None
        self.q_size = self.H * (self.D + self.R)
        self.dkv_size = (self.L + self.R) if self.owns_kv else 0
        self.g_size = self.H * self.Dv
        # One GEMM for q | dkv | gate; rows padded to a multiple of 16
        # so every shape stays on the library's aligned kernels.
        n = self.q_size + self.dkv_size + self.g_size
        self.qdg_proj = ReplicatedLinear(width, _round_up(n, 16),
                                         bias=False, dtype=dtype)
        self.dkv_norm = (RMSNorm(self.L, eps, dtype=torch.float32)
                         if self.owns_kv else None)
        # Per-head expansion weights, laid out for the two batched
        # products: q_abs = q_nope W_uk, out = latent W_uv^T.
        self.w_uk = nn.Parameter(
            torch.empty(self.H, self.D, self.L, dtype=dtype),
            requires_grad=False)
        self.w_uv_t = nn.Parameter(
            torch.empty(self.H, self.L, self.Dv, dtype=dtype),
            requires_grad=False)
        self.o_proj = ReplicatedLinear(self.H * self.Dv, width, bias=False,
                                       dtype=dtype)
        rot = mx["rot"]
        self.attn = LatentAttention(
            self.H, self.D, self.R, self.L, float(mx["scale"]),
            PairwiseRotary(int(rot["dims"]), float(rot["base"])), eps,
            cache_idx, writes_cache=self.owns_kv, has_sink=True)

    def forward(self, h: torch.Tensor, positions: torch.Tensor):
        T = h.shape[0]
        p = self.qdg_proj(h)
        a = self.q_size
        b = a + self.dkv_size
        q = p[:, :a].view(T, self.H, self.D + self.R)
        dkv = p[:, a:b] if self.owns_kv else None
        gate = p[:, b:b + self.g_size]
        self.attn.prepare(
            q, dkv, self.dkv_norm.weight if self.owns_kv else None,
            positions)
        # [H, T, D] x [H, D, L] -> [H, T, L]
        q_abs = torch.bmm(q[..., :self.D].transpose(0, 1), self.w_uk)
        lat = self.attn(q_abs.transpose(0, 1), q[..., self.D:])
        # [H, T, L] x [H, L, Dv] -> [H, T, Dv]
        heads = torch.bmm(lat.transpose(0, 1), self.w_uv_t)
        out = ops.sigmoid_gate_mul(heads.transpose(0, 1), gate)
        return self.o_proj(out)

    def load_parts(self, parts: dict, dtype) -> None:
        need = {"q", "uk", "uv", "sink", "g", "o"}
        if self.owns_kv:
            need |= {"dkv", "dkv.norm"}
        if set(parts) != need:
            raise ValueError(
                f"mixer tensors {sorted(parts)} do not match {sorted(need)}")
        w = self.qdg_proj.weight.data
        w.zero_()
        rows = [parts["q"]] + ([parts["dkv"]] if self.owns_kv else []) \
            + [parts["g"]]
        cat = torch.cat(rows, dim=0).to(dtype)
        w[:cat.shape[0]].copy_(cat)
        if self.owns_kv:
            self.dkv_norm.weight.data.copy_(parts["dkv.norm"].float())
        self.w_uk.data.copy_(
            parts["uk"].to(dtype).view(self.H, self.D, self.L))
        self.w_uv_t.data.copy_(
            parts["uv"].to(dtype).view(self.H, self.Dv, self.L)
            .transpose(1, 2))
        self.attn.sink.data.copy_(parts["sink"].float())
        self.o_proj.weight.data.copy_(parts["o"].to(dtype))


class PapunexMLP(nn.Module):
    """down(relu(up x)^2)."""

    def __init__(self, width: int, ff: int, dtype: torch.dtype):
        super().__init__()
        self.up_proj = ReplicatedLinear(width, ff, bias=False, dtype=dtype)
        self.down_proj = ReplicatedLinear(ff, width, bias=False,
                                          dtype=dtype)

    def forward(self, x):
        return self.down_proj(ops.relu2(self.up_proj(x)))


class PapunexMoE(nn.Module):

    def __init__(self, width: int, ml: dict, dtype: torch.dtype):
        super().__init__()
        r = ml["router"]
        n_exp, top = int(r["experts"]), int(r["top"])
        self.router = SoftmaxTopKRouter(width, n_exp, top,
                                        float(r.get("scale", 1.0)))
        self.experts = FusedMoE(
            n_exp, top, width, int(ml["expert"]["ff"]), renormalize=False,
            activation="relu2", dtype=dtype, learned_router=False,
            gated=False)
        shared = ml.get("shared")
        self.shared = (PapunexMLP(width, int(shared["ff"]), dtype)
                       if shared else None)
        self.shared_gate = (
            nn.Parameter(torch.empty(1, width, dtype=torch.float32),
                         requires_grad=False) if shared else None)

    def forward(self, x):
        weights, ids = self.router(x)
        y = self.experts.run_experts(x, weights, ids)
        if self.shared is not None:
            g = torch.sigmoid(torch.nn.functional.linear(
                x.float(), self.shared_gate))
            y = torch.addcmul(y.float(), self.shared(x).float(), g)
        return y


class PapunexBlock(nn.Module):

    def __init__(self, width: int, entry: dict, eps: float,
                 cache_idx: int, state_idx: int, dtype: torch.dtype):
        super().__init__()
        self.dtype = dtype
        mx = entry["mixer"]
        self.is_attn = entry["type"] == "latent_attention"
        if self.is_attn:
            self.mixer = PapunexLatentMixer(width, mx, eps, cache_idx,
                                            dtype)
        else:
            self.mixer = Mamba2Mixer(
                width, int(mx["heads"]), int(mx["vdim"]), int(mx["state"]),
                int(mx["groups"]), int(mx["conv"]), int(mx["norm_groups"]),
                eps, state_idx, dtype)
        self.norm1 = RMSNorm(width, eps, dtype=torch.float32)
        ml = entry.get("mlp")
        if ml is None:
            self.mlp = None
        elif ml["kind"] == "dense":
            self.mlp = PapunexMLP(width, int(ml["ff"]), dtype)
        else:
            self.mlp = PapunexMoE(width, ml, dtype)
        self.norm2 = (RMSNorm(width, eps, dtype=torch.float32)
                      if ml is not None else None)

    def forward(self, x, xc, positions, next_dtype):
        """x: fp32 stream (updated in place); xc: the same rows in the
        compute dtype. Returns the new xc."""
        y = self.mixer(xc, positions) if self.is_attn else self.mixer(xc)
        if self.mlp is None:
            return self.norm1.add_into(x, y, next_dtype)
        xc = self.norm1.add_into(x, y, self.dtype)
        return self.norm2.add_into(x, self.mlp(xc), next_dtype)


class PapunexModel(nn.Module):

    def __init__(self, config: ModelConfig):
        super().__init__()
        spec = config.spec
        dtype = config.torch_dtype
        if get_tp_world_size() > 1:
            raise NotImplementedError(
                "papunex: tensor parallelism is not implemented")
        self.embed_tokens = VocabParallelEmbedding(
            spec.vocab_size, spec.hidden_size, dtype=dtype)
        self.embedding_scale = spec.embedding_scale
        blocks = []
        n_state = 0
        for i, entry in enumerate(spec.layer_specs):
            # A latent layer's cache index is the layer that owns the
            # keys it reads; the runner allocates per owning layer.
            src = entry["mixer"].get("kv_from")
            blocks.append(PapunexBlock(
                spec.hidden_size, entry, spec.rms_norm_eps,
                cache_idx=i if src is None else int(src),
                state_idx=n_state, dtype=dtype))
            n_state += entry["type"] == "mamba2"
        self.blocks = nn.ModuleList(blocks)
        self.norm = RMSNorm(spec.hidden_size, spec.rms_norm_eps,
                            dtype=torch.float32)
        self.dtype = dtype
        # Set by tests to receive the fp32 stream after every layer.
        self.layer_probe = None

    def forward(self, input_ids, positions, hidden_in=None):
        x = ops.scaled_embedding(input_ids, self.embed_tokens.weight,
                                 self.embedding_scale)
        xc = x if self.dtype == torch.float32 else x.to(self.dtype)
        last = len(self.blocks) - 1
        for i, blk in enumerate(self.blocks):
            # The last layer hands its rows to the final norm, which
            # reads the fp32 stream itself.
            xc = blk(x, xc, positions,
                     torch.float32 if i == last else self.dtype)
            if self.layer_probe is not None:
                self.layer_probe(i, x)
        return self.norm.cast(x, self.dtype)


class PapunexForCausalLM(nn.Module):

    def __init__(self, config: ModelConfig):
        super().__init__()
        spec = config.spec
        self.config = config
        self.model = PapunexModel(config)
        self.lm_head = ParallelLMHead(spec.vocab_size, spec.hidden_size,
                                      dtype=config.torch_dtype)
        self.softcap = spec.logit_softcap

    def forward(self, input_ids, positions, hidden_in=None):
        return self.model(input_ids, positions, hidden_in)

    def compute_logits(self, hidden):
        logits = self.lm_head.compute_logits(hidden)
        if self.softcap > 0:
            logits = ops.logit_softcap(logits, self.softcap)
        return logits

    def finish_dummy_init(self, seed: int) -> None:
        """Random-weight runs: decays and step sizes in a sane range,
        small sinks, unit skip weights."""
        gen = torch.Generator().manual_seed(seed + 29)
        for blk in self.model.blocks:
            if blk.is_attn:
                blk.mixer.attn.sink.data.copy_(
                    torch.randn(blk.mixer.H, generator=gen))
            else:
                mx = blk.mixer
                mx.A_log.data.copy_(
                    torch.rand(mx.heads, generator=gen) * 2.0 - 1.0)
                mx.dt_bias.data.copy_(
                    torch.rand(mx.heads, generator=gen) * 2.0 - 3.0)
                mx.D.data.fill_(1.0)

    def load_hf_weights(self, tensors, config: ModelConfig) -> None:
        """Checkpoint names: embed, final.norm, head, and per layer i
        'l<i>.' + norm1 | norm2 | mix.{q,dkv,dkv.norm,uk,uv,sink,g,o} |
        mix.{in,conv,conv.b,dt_bias,A_log,D,norm,o} | mlp.{up,down} |
        mlp.router | mlp.e<n>.{up,down} | mlp.shared.{up,down,sg}."""
        dtype = config.torch_dtype
        m = self.model
        nl = len(m.blocks)
        mix: list[dict] = [{} for _ in range(nl)]
        experts: list[dict] = [{} for _ in range(nl)]
        seen = set()
        for name, w in tensors:
            seen.add(name)
            if name == "embed":
                m.embed_tokens.load_weight(w.to(dtype))
                continue
            if name == "final.norm":
                m.norm.weight.data.copy_(w.float())
                continue
            if name == "head":
                self.lm_head.load_weight(w.to(dtype))
                continue
            if not (name.startswith("l") and "." in name
                    and name[1:].split(".", 1)[0].isdigit()):
                raise ValueError(f"unknown tensor {name}")
            lid, rest = name[1:].split(".", 1)
            li = int(lid)
            if li >= nl:
                raise ValueError(f"tensor {name}: no such layer")
            blk = m.blocks[li]
            if rest == "norm1":
                blk.norm1.weight.data.copy_(w.float())
            elif rest == "norm2" and blk.norm2 is not None:
                blk.norm2.weight.data.copy_(w.float())
            elif rest.startswith("mix."):
                mix[li][rest[4:]] = w
            elif rest in ("mlp.up", "mlp.down") and isinstance(
                    blk.mlp, PapunexMLP):
                proj = blk.mlp.up_proj if rest == "mlp.up" \
                    else blk.mlp.down_proj
                proj.weight.data.copy_(w.to(dtype))
            elif rest == "mlp.router" and isinstance(blk.mlp, PapunexMoE):
                blk.mlp.router.weight.data.copy_(w.float())
            elif rest.startswith("mlp.shared.") and isinstance(
                    blk.mlp, PapunexMoE) and blk.mlp.shared is not None:
                part = rest[11:]
                if part == "sg":
                    blk.mlp.shared_gate.data.copy_(w.float().view(1, -1))
                elif part == "up":
                    blk.mlp.shared.up_proj.weight.data.copy_(w.to(dtype))
                elif part == "down":
                    blk.mlp.shared.down_proj.weight.data.copy_(w.to(dtype))
                else:
                    raise ValueError(f"unknown tensor {name}")
            elif rest.startswith("mlp.e") and isinstance(
                    blk.mlp, PapunexMoE):
                e, part = rest[5:].split(".", 1)
                experts[li][(int(e), part)] = w.to(dtype)
            else:
                raise ValueError(f"unknown tensor {name}")
        for li, blk in enumerate(m.blocks):
            p = mix[li]
            if blk.is_attn:
                blk.mixer.load_parts(p, dtype)
            else:
                mx = blk.mixer
                need = {"in", "conv", "conv.b", "dt_bias", "A_log", "D",
                        "norm", "o"}
                if set(p) != need:
                    raise ValueError(
                        f"layer {li}: mixer tensors {sorted(p)} do not "
                        f"match {sorted(need)}")
                mx.in_proj.weight.data.copy_(p["in"].to(dtype))
                mx.conv_weight.data.copy_(p["conv"].to(dtype))
                mx.conv_bias.data.copy_(p["conv.b"].to(dtype))
                mx.dt_bias.data.copy_(p["dt_bias"].float())
                mx.A_log.data.copy_(p["A_log"].float())
                mx.D.data.copy_(p["D"].float())
                mx.norm_weight.data.copy_(p["norm"].float())
                mx.out_proj.weight.data.copy_(p["o"].to(dtype))
            if isinstance(blk.mlp, PapunexMoE):
                ex = experts[li]
                n = blk.mlp.experts.num_experts
                try:
                    blk.mlp.experts.load_full_weights(
                        None,
                        torch.stack([ex[(e, "up")] for e in range(n)]),
                        torch.stack([ex[(e, "down")] for e in range(n)]))
                except KeyError as err:
                    raise ValueError(
                        f"layer {li}: missing expert tensor {err}"
                    ) from None
        for need in ("embed", "final.norm", "head"):
            if need not in seen:
                raise ValueError(f"checkpoint lacks tensor {need!r}")

"""Gadilix: a decoder-only stack described layer by layer in its
config.json (sizes, constants and layer order all come from there).

    x = norm_e(embed[token])                              fp32 stream
    per layer:  x += m * norm1(mixer(shift(x)))
                x += m * norm2(ff(x, token))              if it has one
    logits = head(norm_f(x))

- Every norm has a single scalar gain and sits on the sublayer's OUTPUT;
  sublayers read the residual stream itself (layers/layernorm.py
  ScalarRMSNorm). The stream stays fp32 in every compute dtype.
- The mixer reads a token-shifted input (layers/token_shift.py) whose
  one-token carry is per-request, per-layer runner state.
- Mixer "attention": bias-free q/k/v, per-head RMS norm on q and k (one
  [dim] weight shared by all heads), no rotation, GQA, a sliding window
  whose far context is mean-pooled blocks (layers/attention.py
  PooledWindowAttention), a per-head sigmoid output gate that reads the
  same input as the projections, then the output projection. q, k, v
  and the gate come out of ONE fused GEMM.
- Feed-forward: experts chosen by a token-id table with equal weights
  (layers/fused_moe.py TokenTableRouter + FusedMoE.run_experts) plus an
  always-on shared expert; all SwiGLU.
- A layer may borrow another layer's tensors ("weights_of") while
  keeping a cache and shift carry of its own: blocks own parameters,
  layer runs own cache/state indices.

Tensor parallelism is not implemented for this family (tp must be 1).
"""

from __future__ import annotations

import torch
import torch.nn as nn

from vllm_amd import ops
from vllm_amd.config import ModelConfig
from vllm_amd.layers.activation import SiluAndMul
from vllm_amd.layers.attention import PooledWindowAttention
from vllm_amd.layers.embedding import ParallelLMHead, VocabParallelEmbedding
from vllm_amd.layers.fused_moe import FusedMoE, TokenTableRouter
from vllm_amd.layers.layernorm import RMSNorm, ScalarRMSNorm
from vllm_amd.layers.linear import ReplicatedLinear
from vllm_amd.layers.token_shift import TokenShift
from vllm_amd.parallel.state import get_tp_world_size


def _round_up(n: int, m: int) -> int:
    return -(-n // m) * m


class GadilixAttentionMixer(nn.Module):

    def __init__(self, width: int, mx: dict, eps: float,
                 dtype: torch.dtype):
        super().__init__()
        self.H = mx["heads"]
        self.G = mx["kv_heads"]
        self.D = mx["dim"]
        self.Dv = mx["vdim"]
        if self.H % self.G:
            raise ValueError("heads must be a multiple of kv_heads")
        self.q_size = self.H * self.D
        self.k_size = self.G * self.D
        self.v_size = self.G * self.Dv
        # One GEMM for q | k | v | gate; rows padded to a multiple of 16
        # so every GEMM shape stays on the library's aligned kernels.
        n = self.q_size + self.k_size + self.v_size + self.H
        self.qkvg_proj = ReplicatedLinear(width, _round_up(n, 16),
                                          bias=False, dtype=dtype)
        self.o_proj = ReplicatedLinear(self.H * self.Dv, width, bias=False,
                                       dtype=dtype)
        self.q_norm = RMSNorm(self.D, eps, dtype=dtype)
        self.k_norm = RMSNorm(self.D, eps, dtype=dtype)
        self.attn = PooledWindowAttention(
            self.H, self.D, self.Dv, scale=float(mx["scale"]),
            num_kv_heads=self.G, window=int(mx["mask"]["size"]),
            pool=int(mx["mask"]["pool"]))

    def forward(self, h: torch.Tensor, cache_idx: int) -> torch.Tensor:
        T = h.shape[0]
        qkvg = self.qkvg_proj(h)
        a = self.q_size
        b = a + self.k_size
        c = b + self.v_size
        q = qkvg[:, :a].view(T, self.H, self.D)
        k = qkvg[:, a:b].view(T, self.G, self.D)
        v = qkvg[:, b:c].view(T, self.G, self.Dv)
        gate = qkvg[:, c:c + self.H]
        out = self.attn(q, k, v, gate, cache_idx,
                        qk_norm=(self.q_norm.weight, self.k_norm.weight,
                                 self.q_norm.eps))
        return self.o_proj(out)

    def load_fused(self, q, k, v, g) -> None:
        w = self.qkvg_proj.weight.data
        w.zero_()
        w[:self.q_size + self.k_size + self.v_size + self.H].copy_(
            torch.cat([q, k, v, g], dim=0))


class GadilixExpert(nn.Module):
    """Dense SwiGLU expert: down(silu(gate x) * up x)."""

    def __init__(self, width: int, ff: int, dtype: torch.dtype):
        super().__init__()
        self.ff = ff
        self.gate_up_proj = ReplicatedLinear(width, 2 * ff, bias=False,
                                             dtype=dtype)
        self.down_proj = ReplicatedLinear(ff, width, bias=False,
                                          dtype=dtype)
        self.act_fn = SiluAndMul()

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_up_proj(x)))


class GadilixMoE(nn.Module):

    def __init__(self, width: int, vocab: int, ml: dict,
                 dtype: torch.dtype):
        super().__init__()
        n_exp = int(ml["router"]["experts"])
        top = int(ml["router"]["top"])
        self.router = TokenTableRouter(vocab, top)
        self.experts = FusedMoE(
            n_exp, top, width, int(ml["expert"]["ff"]), renormalize=False,
            activation="silu", dtype=dtype, learned_router=False)
        shared = ml.get("shared")
        self.shared = (GadilixExpert(width, int(shared["ff"]), dtype)
                       if shared else None)

    def forward(self, x, input_ids):
        weights, ids = self.router(input_ids)
        y = self.experts.run_experts(x, weights, ids)
        if self.shared is not None:
            y = y + self.shared(x)
        return y


class GadilixBlock(nn.Module):
    """Parameters of one layer (mixer, feed-forward, norms, shift).
    Stateless across layer runs: cache and carry indices come in with
    each call, so several layer runs can share one block."""

    def __init__(self, width: int, vocab: int, entry: dict, eps: float,
                 mult: float, dtype: torch.dtype):
        super().__init__()
        self.mult = mult
        self.dtype = dtype
        self.shift = TokenShift(width)
        self.mixer = GadilixAttentionMixer(width, entry["mixer"], eps,
                                           dtype)
        self.norm1 = ScalarRMSNorm(eps)
        ml = entry.get("mlp")
        self.mlp = GadilixMoE(width, vocab, ml, dtype) if ml else None
        self.norm2 = ScalarRMSNorm(eps) if ml else None

    def forward(self, x: torch.Tensor, input_ids: torch.Tensor,
                run_idx: int) -> torch.Tensor:
        h = self.shift(x, run_idx, self.dtype)
        y = self.mixer(h, run_idx)
        xc = self.norm1.add_into(x, y, self.mult, self.dtype)
        if self.mlp is not None:
            y = self.mlp(xc, input_ids)
            self.norm2.add_into(x, y, self.mult)
        return x


class GadilixModel(nn.Module):

    def __init__(self, config: ModelConfig):
        super().__init__()
        spec = config.spec
        dtype = config.torch_dtype
        if get_tp_world_size() > 1:
            raise NotImplementedError(
                "gadilix: tensor parallelism is not implemented")
        self.embed_tokens = VocabParallelEmbedding(
            spec.vocab_size, spec.hidden_size, dtype=dtype)
        self.embed_norm = ScalarRMSNorm(spec.rms_norm_eps)
        blocks = {}
        for i, entry in enumerate(spec.layer_specs):
            if entry.get("weights_of") is None:
                blocks[str(i)] = GadilixBlock(
                    spec.hidden_size, spec.vocab_size, entry,
                    spec.rms_norm_eps, spec.residual_mult, dtype)
        # Keys are the config's layer indices, so parameter names keep
        # them ("blocks.3.mixer...").
        self.blocks = nn.ModuleDict(blocks)
        # Layer run i -> the block that holds its parameters.
        self.block_of = [
            str(e["weights_of"] if e.get("weights_of") is not None else i)
            for i, e in enumerate(spec.layer_specs)]
        self.norm = ScalarRMSNorm(spec.rms_norm_eps)
        self.dtype = dtype

    def forward(self, input_ids, positions, hidden_in=None):
        x = self.embed_norm(self.embed_tokens(input_ids))
        for run_idx, key in enumerate(self.block_of):
            x = self.blocks[key](x, input_ids, run_idx)
        return self.norm(x, out_dtype=self.dtype)


class GadilixForCausalLM(nn.Module):

    def __init__(self, config: ModelConfig):
        super().__init__()
        spec = config.spec
        self.config = config
        self.model = GadilixModel(config)
        self.lm_head = ParallelLMHead(spec.vocab_size, spec.hidden_size,
                                      dtype=config.torch_dtype)

    def forward(self, input_ids, positions, hidden_in=None):
        return self.model(input_ids, positions, hidden_in)

    def compute_logits(self, hidden):
        return self.lm_head.compute_logits(hidden)

    def finish_dummy_init(self, seed: int) -> None:
        """Random-weight runs: unit scalar gains, blend factors in
        [0, 1), distinct random experts per token id."""
        gen = torch.Generator().manual_seed(seed + 17)
        m = self.model
        m.embed_norm.gain.data.fill_(1.0)
        m.norm.gain.data.fill_(1.0)
        for blk in m.blocks.values():
            blk.norm1.gain.data.fill_(1.0)
            blk.shift.mu.data.copy_(
                torch.rand(blk.shift.mu.shape, generator=gen))
            if blk.mlp is None:
                continue
            blk.norm2.gain.data.fill_(1.0)
            tab = blk.mlp.router.table
            n_exp = blk.mlp.experts.num_experts
            scores = torch.rand(tab.shape[0], n_exp, generator=gen)
            tab.copy_(scores.topk(tab.shape[1], dim=1).indices
                      .to(torch.int32))

    def load_hf_weights(self, tensors, config: ModelConfig) -> None:
        """Checkpoint names: embed, embed.norm, final.norm, head, and per
        layer i with tensors of its own 'l<i>.' + norm1 | norm2 | shift |
        mix.{q,k,v,g,o} | mix.{q,k}.norm | mlp.table |
        mlp.e<n>.{gate,up,down} | mlp.shared.{gate,up,down}."""
        dtype = config.torch_dtype
        m = self.model
        mix_parts: dict[str, dict] = {}
        experts: dict[str, dict] = {}
        shared: dict[str, dict] = {}
        seen = set()
        for name, w in tensors:
            seen.add(name)
            if name == "embed":
                m.embed_tokens.load_weight(w.to(dtype))
            elif name == "embed.norm":
                m.embed_norm.gain.data.copy_(w.float())
            elif name == "final.norm":
                m.norm.gain.data.copy_(w.float())
            elif name == "head":
                self.lm_head.load_weight(w.to(dtype))
            elif name.startswith("l") and "." in name:
                lid, rest = name[1:].split(".", 1)
                if lid not in m.blocks:
                    raise ValueError(f"tensor {name}: no such layer")
                blk = m.blocks[lid]
                if rest == "norm1":
                    blk.norm1.gain.data.copy_(w.float())
                elif rest == "norm2":
                    blk.norm2.gain.data.copy_(w.float())
                elif rest == "shift":
                    blk.shift.mu.data.copy_(w.float())
                elif rest == "mix.q.norm":
                    blk.mixer.q_norm.weight.data.copy_(w.to(dtype))
                elif rest == "mix.k.norm":
                    blk.mixer.k_norm.weight.data.copy_(w.to(dtype))
                elif rest == "mix.o":
                    blk.mixer.o_proj.weight.data.copy_(w.to(dtype))
                elif rest in ("mix.q", "mix.k", "mix.v", "mix.g"):
                    mix_parts.setdefault(lid, {})[rest[4:]] = w.to(dtype)
                elif rest == "mlp.table":
                    blk.mlp.router.table.copy_(w.to(torch.int32))
                elif rest.startswith("mlp.shared."):
                    shared.setdefault(lid, {})[rest[11:]] = w.to(dtype)
                elif rest.startswith("mlp.e"):
                    e, part = rest[5:].split(".", 1)
                    experts.setdefault(lid, {})[(int(e), part)] = \
                        w.to(dtype)
                else:
                    raise ValueError(f"unknown tensor {name}")
            else:
                raise ValueError(f"unknown tensor {name}")
        for lid, blk in m.blocks.items():
            p = mix_parts.get(lid, {})
            if set(p) != {"q", "k", "v", "g"}:
                raise ValueError(f"layer {lid}: incomplete mixer tensors")
            blk.mixer.load_fused(p["q"], p["k"], p["v"], p["g"])
            if blk.mlp is None:
                continue
            ex = experts.get(lid, {})
            n = blk.mlp.experts.num_experts
            try:
                blk.mlp.experts.load_full_weights(
                    torch.stack([ex[(e, "gate")] for e in range(n)]),
                    torch.stack([ex[(e, "up")] for e in range(n)]),
                    torch.stack([ex[(e, "down")] for e in range(n)]))
            except KeyError as err:
                raise ValueError(
                    f"layer {lid}: missing expert tensor {err}") from None
            if blk.mlp.shared is not None:
                sh = shared.get(lid, {})
                blk.mlp.shared.gate_up_proj.weight.data.copy_(
                    torch.cat([sh["gate"], sh["up"]], dim=0))
                blk.mlp.shared.down_proj.weight.data.copy_(sh["down"])
        for need in ("embed", "embed.norm", "final.norm", "head"):
            if need not in seen:
                raise ValueError(f"checkpoint lacks tensor {need!r}")

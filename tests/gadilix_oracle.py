"""Plain, slow, whole-sequence implementation of the Gadilix design,
one function per mechanism, written from its equations only. It shares
no code with vllm_amd: tests compare the engine against it.

Notation: x residual stream [T, W]; m residual multiplier; eps norm
epsilon; for attention H query heads, G key/value heads, d key width,
dv value width, Wn window size, P pooled block size.
"""

from __future__ import annotations

import json
import math
import os

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """One gain for all coordinates."""
    return unit_rms(x, eps) * g


def token_shift(h, mu):
    """h~[t] = h[t] + (h[t-1] - h[t]) * mu, h[-1] = 0."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    return h + (prev - h) * mu


def visible_keys(i, Wn, P):
    """(window positions, pooled block ids) that position i sees."""
    toks = [j for j in range(0, i + 1) if 0 <= i - j < Wn]
    blocks = []
    b = 0
    while b * P + P - 1 <= i - Wn:
        blocks.append(b)
        b += 1
    return toks, blocks


def pooled_window_attention(q, k, v, scale, Wn, P):
    """q [T,H,d], k [T,G,d], v [T,G,dv] -> [T,H,dv]; positions do not
    enter the scores."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2])
    for i in range(T):
        toks, blocks = visible_keys(i, Wn, P)
        for h in range(H):
            g = h // (H // G)
            keys = [k[j, g] for j in toks]
            vals = [v[j, g] for j in toks]
            for b in blocks:
                keys.append(k[b * P:b * P + P, g].mean(0))
                vals.append(v[b * P:b * P + P, g].mean(0))
            K = torch.stack(keys)
            V = torch.stack(vals)
            w = torch.softmax((K @ q[i, h]) * scale, dim=0)
            out[i, h] = w @ V
    return out


def attention_mixer(h, wt, pre, mx, eps):
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = (h @ wt[pre + "q"].T).view(T, H, d)
    k = (h @ wt[pre + "k"].T).view(T, G, d)
    v = (h @ wt[pre + "v"].T).view(T, G, dv)
    q = unit_rms(q, eps) * wt[pre + "q.norm"]
    k = unit_rms(k, eps) * wt[pre + "k.norm"]
    o = pooled_window_attention(q, k, v, mx["scale"], mx["mask"]["size"],
                                mx["mask"]["pool"])
    gate = torch.sigmoid(h @ wt[pre + "g"].T)          # [T, H]
    o = o * gate.unsqueeze(-1)
    return o.reshape(T, H * dv) @ wt[pre + "o"].T


def swiglu(x, wt, pre):
    a = x @ wt[pre + "gate"].T
    return ((a * torch.sigmoid(a)) * (x @ wt[pre + "up"].T)) \
        @ wt[pre + "down"].T


def table_moe(x, tokens, wt, pre, ml):
    top = ml["router"]["top"]
    y = torch.zeros_like(x)
    table = wt[pre + "table"]
    for t, tok in enumerate(tokens):
        for e in table[tok].tolist():
            y[t] += swiglu(x[t:t + 1], wt, f"{pre}e{e}.")[0] / top
    if ml.get("shared"):
        y = y + swiglu(x, wt, pre + "shared.")
    return y


def forward(cfg, wt, tokens, layer_outputs=None):
    """Logits [T, vocab] of a whole sequence."""
    eps = cfg["norm"]["eps"]
    m = cfg["residual_mult"]
    ids = torch.tensor(tokens)
    x = scalar_norm(wt["embed"][ids], wt["embed.norm"], eps)
    for i, layer in enumerate(cfg["layers"]):
        j = layer.get("weights_of")
        p = f"l{i if j is None else j}."
        h = token_shift(x, wt[p + "shift"])
        y = attention_mixer(h, wt, p + "mix.", layer["mixer"], eps)
        x = x + m * scalar_norm(y, wt[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            y = table_moe(x, tokens, wt, p + "mlp.", layer["mlp"])
            x = x + m * scalar_norm(y, wt[p + "norm2"], eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return scalar_norm(x, wt["final.norm"], eps) @ wt["head"].T


# ----------------------------------------------------------------------
# Random models in the checkpoint layout.

def layer_entry(heads=4, kv_heads=2, dim=8, vdim=8, window=6, pool=3,
                scale=None, experts=4, top=2, ff=16, shared_ff=24,
                mlp=True, weights_of=None):
    entry = {
        "type": "attention",
        "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                  "vdim": vdim, "scale": scale or 1.0 / math.sqrt(dim),
                  "mask": {"size": window, "pool": pool}},
        "mlp": ({"kind": "moe", "expert": {"ff": ff},
                 "router": {"experts": experts, "top": top},
                 "shared": {"ff": shared_ff}} if mlp else None),
    }
    if weights_of is not None:
        entry["weights_of"] = weights_of
    return entry


def make_config(layers, vocab=40, width=32, eps=1e-5, residual_mult=0.5):
    return {"architecture": "Gadilix", "vocab": vocab, "width": width,
            "residual_mult": residual_mult, "norm": {"eps": eps},
            "layers": layers}


def random_weights(cfg, seed=0, sharp=3.0):
    """bf16-representable fp32 weights. `sharp` scales q/k so that the
    softmax is far from uniform and a wrong key set changes the output
    visibly."""
    gen = torch.Generator().manual_seed(seed)

    def mat(o, i, s=1.0):
        w = torch.randn(o, i, generator=gen) * s / math.sqrt(i)
        return w.bfloat16().float()

    def vec(n, lo, hi):
        return (torch.rand(n, generator=gen) * (hi - lo) + lo) \
            .bfloat16().float()

    V, W = cfg["vocab"], cfg["width"]
    wt = {"embed": mat(V, W, math.sqrt(W)), "embed.norm": vec(1, .8, 1.2)[0],
          "final.norm": vec(1, .8, 1.2)[0], "head": mat(V, W)}
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p = f"l{i}."
        mx = layer["mixer"]
        H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        wt[p + "norm1"] = vec(1, .8, 1.2)[0]
        wt[p + "shift"] = vec(W, 0.0, 1.0)
        wt[p + "mix.q"] = mat(H * d, W, sharp)
        wt[p + "mix.k"] = mat(G * d, W, sharp)
        wt[p + "mix.v"] = mat(G * dv, W)
        wt[p + "mix.g"] = mat(H, W, 2.0)
        wt[p + "mix.o"] = mat(W, H * dv)
        wt[p + "mix.q.norm"] = vec(d, .5, 1.5)
        wt[p + "mix.k.norm"] = vec(d, .5, 1.5)
        ml = layer.get("mlp")
        if ml is None:
            continue
        wt[p + "norm2"] = vec(1, .8, 1.2)[0]
        E, top, ff = ml["router"]["experts"], ml["router"]["top"], \
            ml["expert"]["ff"]
        for e in range(E):
            wt[f"{p}mlp.e{e}.gate"] = mat(ff, W)
            wt[f"{p}mlp.e{e}.up"] = mat(ff, W)
            wt[f"{p}mlp.e{e}.down"] = mat(W, ff)
        scores = torch.rand(V, E, generator=gen)
        wt[p + "mlp.table"] = scores.topk(top, dim=1).indices \
            .to(torch.int32)
        if ml.get("shared"):
            sf = ml["shared"]["ff"]
            wt[p + "mlp.shared.gate"] = mat(sf, W)
            wt[p + "mlp.shared.up"] = mat(sf, W)
            wt[p + "mlp.shared.down"] = mat(W, sf)
    return wt


def save_model(path, cfg, wt):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: (v.contiguous() if v.dtype == torch.int32
                   else v.bfloat16().contiguous())
               for k, v in wt.items()},
              os.path.join(path, "model.safetensors"))
    return path

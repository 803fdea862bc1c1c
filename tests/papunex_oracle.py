"""Slow reference for the Papunex family, one function per mechanism,
written from the family's equations with plain fp32 torch and Python
loops. Nothing here is shared with vllm_amd's model, ops or kernels.

A model is (cfg, W): cfg is the config.json dict, W maps checkpoint
tensor names to fp32 tensors. `forward` runs a whole sequence at once
and can return the residual stream after every layer.
"""

from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotate_pairs(v, pos, base, dims):
    """v [..., n]: coordinates (2i, 2i+1), i < dims/2, turn by the angle
    pos * base**(-2i/dims); coordinates >= dims stay."""
    out = v.clone()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, w = v[..., 2 * i].clone(), v[..., 2 * i + 1].clone()
        out[..., 2 * i] = u * c - w * s
        out[..., 2 * i + 1] = w * c + u * s
    return out


def latent_kv(h, mx, W, pre, eps):
    """Per token: latent c [T, L] (normed) and the shared rotated key
    part kr [T, R] (rotated by position)."""
    L, R = mx["kv_rank"], mx["rot_dim"]
    T = h.shape[0]
    d = h @ W[pre + "dkv"].T
    c = rms(d[:, :L], eps) * W[pre + "dkv.norm"]
    kr = torch.stack([
        rotate_pairs(d[t, L:L + R], t, mx["rot"]["base"], mx["rot"]["dims"])
        for t in range(T)])
    return c, kr


def latent_attention(h, mx, W, pre, eps, shared=None):
    """Whole-sequence causal latent attention with a per-head sink in
    the softmax denominator and a sigmoid output gate.
    shared = (c, kr) of another layer when this one borrows its keys.
    Returns (out [T, width], (c, kr))."""
    H, D, R, Dv = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"]
    L = mx["kv_rank"]
    T = h.shape[0]
    q = (h @ W[pre + "q"].T).view(T, H, D + R)
    c, kr = shared if shared is not None else latent_kv(h, mx, W, pre, eps)
    k_nope = (c @ W[pre + "uk"].T).view(T, H, D)
    v = (c @ W[pre + "uv"].T).view(T, H, Dv)
    sink = W[pre + "sink"]
    heads = torch.zeros(T, H, Dv)
    for t in range(T):
        for hh in range(H):
            qn = q[t, hh, :D]
            qr = rotate_pairs(q[t, hh, D:], t, mx["rot"]["base"],
                              mx["rot"]["dims"])
            s = (k_nope[:t + 1, hh] @ qn + kr[:t + 1] @ qr) * mx["scale"]
            m = max(float(s.max()), float(sink[hh]))
            e = torch.exp(s - m)
            den = e.sum() + math.exp(float(sink[hh]) - m)
            heads[t, hh] = (e[:, None] * v[:t + 1, hh]).sum(0) / den
    gate = torch.sigmoid(h @ W[pre + "g"].T)
    out = (heads.reshape(T, H * Dv) * gate) @ W[pre + "o"].T
    return out, (c, kr)


def causal_conv_silu(u, w, b):
    """u [T, C], w [C, K] (last column = current token), zeros before
    the start."""
    T, C = u.shape
    K = w.shape[1]
    out = torch.zeros(T, C)
    for t in range(T):
        acc = b.clone()
        for j in range(K):
            src = t - (K - 1) + j
            if src >= 0:
                acc = acc + w[:, j] * u[src]
        out[t] = acc
    return out * torch.sigmoid(out)


def ssd_scan(x, B, C, dt, A, D, groups):
    """x [T, Hm, P], B/C [T, G, N], dt [T, Hm] (already positive),
    A [Hm] > 0, D [Hm]. State per head [N, P], zero at the start."""
    T, Hm, P = x.shape
    N = B.shape[-1]
    per = Hm // groups
    y = torch.zeros(T, Hm, P)
    for hh in range(Hm):
        g = hh // per
        S = torch.zeros(N, P)
        for t in range(T):
            S = math.exp(-float(A[hh]) * float(dt[t, hh])) * S \
                + float(dt[t, hh]) * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S.T @ C[t, g] + D[hh] * x[t, hh]
    return y


def mamba2(h, mx, W, pre, eps):
    Hm, P, N, G = mx["heads"], mx["vdim"], mx["state"], mx["groups"]
    inner = Hm * P
    T = h.shape[0]
    p = h @ W[pre + "in"].T
    z = p[:, :inner]
    xbc = p[:, inner:2 * inner + 2 * G * N]
    dt = p[:, 2 * inner + 2 * G * N:]
    xbc = causal_conv_silu(xbc, W[pre + "conv"], W[pre + "conv.b"])
    x = xbc[:, :inner].reshape(T, Hm, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = torch.nn.functional.softplus(dt + W[pre + "dt_bias"])
    y = ssd_scan(x, B, C, dt, torch.exp(W[pre + "A_log"]), W[pre + "D"], G)
    y = y.reshape(T, inner) * (z * torch.sigmoid(z))
    ng = mx["norm_groups"]
    y = rms(y.view(T, ng, inner // ng), eps).reshape(T, inner)
    return (y * W[pre + "norm"]) @ W[pre + "o"].T


def relu2_mlp(h, up, down):
    a = torch.relu(h @ up.T)
    return (a * a) @ down.T


def moe(h, ml, W, pre):
    r = ml["router"]
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ W[pre + "router"].T, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: -float(s[t, e]))[:top]
        tot = sum(float(s[t, e]) for e in order) + 1e-20
        for e in order:
            wgt = float(s[t, e]) / tot * r["scale"]
            out[t] += wgt * relu2_mlp(
                h[t:t + 1], W[f"{pre}e{e}.up"], W[f"{pre}e{e}.down"])[0]
    if ml.get("shared"):
        sg = torch.sigmoid(h @ W[pre + "shared.sg"].T)     # [T, 1]
        out = out + sg * relu2_mlp(h, W[pre + "shared.up"],
                                   W[pre + "shared.down"])
    return out


def feed_forward(h, ml, W, pre):
    if ml["kind"] == "dense":
        return relu2_mlp(h, W[pre + "up"], W[pre + "down"])
    return moe(h, ml, W, pre)


def forward(cfg, W, tokens, return_layers=False):
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    kv = {}
    per_layer = []
    for i, lay in enumerate(cfg["layers"]):
        mx = lay["mixer"]
        pre = f"l{i}.mix."
        if lay["type"] == "mamba2":
            y = mamba2(x, mx, W, pre, eps)
        else:
            src = mx.get("kv_from")
            y, own = latent_attention(
                x, mx, W, pre, eps,
                shared=kv[src] if src is not None else None)
            if src is None:
                kv[i] = own
        x = x + rms(y, eps) * W[f"l{i}.norm1"]
        if lay.get("mlp"):
            y = feed_forward(x, lay["mlp"], W, f"l{i}.mlp.")
            x = x + rms(y, eps) * W[f"l{i}.norm2"]
        per_layer.append(x.clone())
    logits = (rms(x, eps) * W["final.norm"]) @ W["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return (logits, torch.stack(per_layer)) if return_layers else logits


# ---------------------------------------------------------------------
# Test models: configurations, random weights, files on disk.

def latent_entry(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=8,
                 rot_dims=None, base=100.0, scale=None, kv_from=None,
                 mlp="dense", ff=16, experts=4, top=2, router_scale=1.0,
                 shared_ff=8):
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
          "kv_rank": kv_rank,
          "rot": {"base": base,
                  "dims": rot_dim if rot_dims is None else rot_dims},
          "scale": scale if scale is not None
          else 1.0 / math.sqrt(dim + rot_dim)}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mx,
            "mlp": mlp_entry(mlp, ff, experts, top, router_scale,
                             shared_ff)}


def mamba_entry(heads=4, vdim=8, state=8, groups=2, conv=4, norm_groups=2,
                mlp="dense", ff=16, experts=4, top=2, router_scale=1.0,
                shared_ff=8):
    mx = {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
          "conv": conv, "norm_groups": norm_groups}
    return {"type": "mamba2", "mixer": mx,
            "mlp": mlp_entry(mlp, ff, experts, top, router_scale,
                             shared_ff)}


def mlp_entry(kind, ff, experts, top, router_scale, shared_ff):
    if kind is None:
        return None
    if kind == "dense":
        return {"kind": "dense", "ff": ff}
    out = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "top": top,
                      "scale": router_scale}}
    if shared_ff:
        out["shared"] = {"ff": shared_ff}
    return out


def make_config(layers, vocab=48, width=24, eps=1e-5, embed_scale=2.0,
                softcap=20.0):
    return {"architecture": "Papunex", "vocab": vocab, "width": width,
            "embedding": {"scale": embed_scale}, "norm": {"eps": eps},
            "logit_softcap": softcap, "layers": layers}


def random_weights(cfg, seed=0):
    """fp32 tensors whose values are exactly representable in bf16."""
    gen = torch.Generator().manual_seed(seed)
    Wd = cfg["width"]

    def mat(o, i, gain=1.0):
        w = torch.randn(o, i, generator=gen) * gain / math.sqrt(i)
        return w.bfloat16().float()

    def vec(n, lo, hi):
        return (torch.rand(n, generator=gen) * (hi - lo) + lo) \
            .bfloat16().float()

    W = {"embed": (torch.randn(cfg["vocab"], Wd, generator=gen) * 0.5)
         .bfloat16().float(),
         "final.norm": vec(Wd, 0.5, 1.5),
         "head": mat(cfg["vocab"], Wd, 2.0)}
    for i, lay in enumerate(cfg["layers"]):
        mx, pre = lay["mixer"], f"l{i}.mix."
        W[f"l{i}.norm1"] = vec(Wd, 0.5, 1.5)
        if lay["type"] == "latent_attention":
            H, D, R = mx["heads"], mx["dim"], mx["rot_dim"]
            Dv, L = mx["vdim"], mx["kv_rank"]
            W[pre + "q"] = mat(H * (D + R), Wd, 2.0)
            if mx.get("kv_from") is None:
                W[pre + "dkv"] = mat(L + R, Wd, 2.0)
                W[pre + "dkv.norm"] = vec(L, 0.5, 1.5)
            W[pre + "uk"] = mat(H * D, L, 2.0)
            W[pre + "uv"] = mat(H * Dv, L)
            W[pre + "sink"] = vec(H, -1.0, 2.0)
            W[pre + "g"] = mat(H * Dv, Wd)
            W[pre + "o"] = mat(Wd, H * Dv)
        else:
            Hm, P, N, G = (mx["heads"], mx["vdim"], mx["state"],
                           mx["groups"])
            inner, ch = Hm * P, Hm * P + 2 * G * N
            W[pre + "in"] = mat(2 * inner + 2 * G * N + Hm, Wd)
            W[pre + "conv"] = mat(ch, mx["conv"], 1.5)
            W[pre + "conv.b"] = vec(ch, -0.2, 0.2)
            W[pre + "dt_bias"] = vec(Hm, -2.0, 0.5)
            W[pre + "A_log"] = vec(Hm, -1.5, 0.5)
            W[pre + "D"] = vec(Hm, 0.5, 1.5)
            W[pre + "norm"] = vec(inner, 0.5, 1.5)
            W[pre + "o"] = mat(Wd, inner)
        ml = lay.get("mlp")
        if ml is None:
            continue
        W[f"l{i}.norm2"] = vec(Wd, 0.5, 1.5)
        pre = f"l{i}.mlp."
        if ml["kind"] == "dense":
            W[pre + "up"] = mat(ml["ff"], Wd, 1.5)
            W[pre + "down"] = mat(Wd, ml["ff"], 1.5)
            continue
        W[pre + "router"] = mat(ml["router"]["experts"], Wd, 3.0)
        for e in range(ml["router"]["experts"]):
            W[f"{pre}e{e}.up"] = mat(ml["expert"]["ff"], Wd, 1.5)
            W[f"{pre}e{e}.down"] = mat(Wd, ml["expert"]["ff"], 1.5)
        if ml.get("shared"):
            W[pre + "shared.up"] = mat(ml["shared"]["ff"], Wd, 1.5)
            W[pre + "shared.down"] = mat(Wd, ml["shared"]["ff"], 1.5)
            W[pre + "shared.sg"] = mat(1, Wd, 2.0)
    return W


def save_model(path, cfg, W):
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in W.items()},
              os.path.join(path, "model.safetensors"))
    return path

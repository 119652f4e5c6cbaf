"""Slow float64 oracle of the Pinavik decoder, written from its equations: one function per mechanism, whole
sequences at once, plain loops for the recurrences. It shares no code with the framework (no ops, no engine, no model
class); it reads the checkpoint layout (tensor names) and the config dictionary only.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def root_mean_square_div(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def centred_norm(x, w, eps):
    return root_mean_square_div(x, eps) * (1.0 + w)


def attention_mixer(h, W, p, m, eps):
    """h [T, width] -> [T, width]. Whole-projection q / k norms, capped scores, log-distance penalty, window."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (root_mean_square_div(h @ W[p + "q"].T, eps) * W[p + "q.norm"]).reshape(T, H, dk)
    k = (root_mean_square_div(h @ W[p + "k"].T, eps) * W[p + "k.norm"]).reshape(T, G, dk)
    v = (h @ W[p + "v"].T).reshape(T, G, dv)
    cap = m.get("softcap")
    win = (m.get("mask") or {}).get("size")
    heads = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        for hh in range(H):
            g = hh // (H // G)
            lo = 0 if not win else max(0, i - win + 1)
            sc = torch.empty(i - lo + 1, dtype=F64)
            for n, j in enumerate(range(lo, i + 1)):
                s = float(q[i, hh] @ k[j, g]) * m["scale"]
                if cap:
                    s = cap * math.tanh(s / cap)
                s -= float(W[p + "r1"][hh]) * math.log(1.0 + float(W[p + "r2"][hh]) * (i - j))
                sc[n] = s
            pr = torch.softmax(sc, 0)
            heads[i, hh] = pr @ v[lo:i + 1, g]
    gate = torch.sigmoid(h @ W[p + "g"].T)
    return (heads.reshape(T, H * dv) * gate) @ W[p + "o"].T


def wkv_mixer(h, W, p, m, eps):
    T, D = h.shape
    H, d = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, D, dtype=F64), h[:-1]])

    def mixed(s):
        return h + (prev - h) * W[p + "mu." + s]

    r = (mixed("r") @ W[p + "r"].T).reshape(T, H, d)
    k = (mixed("k") @ W[p + "k"].T).reshape(T, H, d)
    v = (mixed("v") @ W[p + "v"].T).reshape(T, H, d)
    gate = torch.nn.functional.silu(mixed("g") @ W[p + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mixed("w") @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])).reshape(T, H, d)
    u = W[p + "u"].reshape(H, d)
    out = torch.zeros(T, H, d, dtype=F64)
    for hh in range(H):
        S = torch.zeros(d, d, dtype=F64)
        for t in range(T):
            kv = torch.outer(k[t, hh], v[t, hh])
            out[t, hh] = (S + u[hh][:, None] * kv).T @ r[t, hh]
            S = decay[t, hh][:, None] * S + kv
    out = root_mean_square_div(out, eps).reshape(T, H * d) * W[p + "norm"] * gate
    return out @ W[p + "o"].T


def short_conv_silu(x, taps):
    """x [T, C], taps [C, K] (last column = current token), zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for i in range(K):
            src = t - (K - 1) + i
            if src >= 0:
                y[t] += x[src] * taps[:, i]
    return torch.nn.functional.silu(y)


def channel_delta_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(h @ W[p + "q"].T, W[p + "q.conv"]).reshape(T, G, dk)
    k = short_conv_silu(h @ W[p + "k"].T, W[p + "k.conv"]).reshape(T, G, dk)
    v = short_conv_silu(h @ W[p + "v"].T, W[p + "v.conv"]).reshape(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    pre = ((h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]).reshape(T, H, dk)
    g = torch.exp(-torch.exp(W[p + "A_log"])[None, :, None] * torch.nn.functional.softplus(pre))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        kh = hh // (H // G)
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = g[t, hh][:, None] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            out[t, hh] = S.T @ q[t, kh]
    out = root_mean_square_div(out, eps) * W[p + "norm"]
    gate = torch.sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T).reshape(T, H, dv)
    return (out * gate).reshape(T, H * dv) @ W[p + "o"].T


def polynorm_ff(h, W, p, eps):
    z = h @ W[p + "up"].T
    a, b, c, e = [float(x) for x in W[p + "act"]]
    y = a * root_mean_square_div(z, eps) + b * root_mean_square_div(z ** 2, eps) + c * root_mean_square_div(z ** 3, eps) + e
    return y @ W[p + "down"].T


MIXER = {"attention": attention_mixer, "wkv": wkv_mixer, "channel_delta": channel_delta_mixer}


def forward(cfg: dict, sd: dict, tokens, residuals: list | None = None) -> torch.Tensor:
    """cfg: the config.json dictionary; sd: checkpoint tensors. Returns float64 logits [T, vocab]."""
    W = {k: v.to(F64) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    mult = cfg["residual_mult"]
    x0 = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    layers = cfg["layers"]
    loop = cfg.get("loop") or None

    def layer(i, x):
        l, p = layers[i], f"l{i}."
        x = x + mult * MIXER[l["type"]](centred_norm(x, W[p + "norm1"], eps), W, p + "mix.", l["mixer"], eps)
        if l.get("mlp") is not None:
            x = x + mult * polynorm_ff(centred_norm(x, W[p + "norm2"], eps), W, p + "mlp.", eps)
        if residuals is not None:
            residuals.append(x)
        return x

    x = x0
    if not loop or not loop.get("times"):
        for i in range(len(layers)):
            x = layer(i, x)
    else:
        for i in range(loop["start"]):
            x = layer(i, x)
        for t in range(loop["times"]):
            x = torch.cat([x, x0], -1) @ W["loop.in"].T + W["loop.step"][t]
            for i in range(loop["start"], loop["stop"]):
                x = layer(i, x)
        for i in range(loop["stop"], len(layers)):
            x = layer(i, x)
    return centred_norm(x, W["final.norm"], eps) @ W["head"].T


def random_checkpoint(cfg: dict, seed: int = 0, slow_decay: bool = False) -> dict:
    """Random bf16-representable checkpoint for a config dictionary. slow_decay: recurrent states forget slowly, so a
    token hundreds of positions back still shows in the output."""
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]

    def rn(*s, std=1.0):
        return (torch.randn(*s, generator=g) * std).to(torch.bfloat16).float()

    def un(*s, lo=0.0, hi=1.0):
        return (torch.rand(*s, generator=g) * (hi - lo) + lo).to(torch.bfloat16).float()

    def lin(o, i):
        return rn(o, i, std=i ** -0.5)

    sd = {"embed": rn(cfg["vocab"], D, std=1.0 / cfg["embedding"]["scale"]), "head": lin(cfg["vocab"], D),
          "final.norm": rn(D, std=0.2)}
    loop = cfg.get("loop")
    if loop and loop.get("times"):
        sd["loop.in"] = lin(D, 2 * D) * 1.5
        sd["loop.in"] = sd["loop.in"].to(torch.bfloat16).float()
        sd["loop.step"] = rn(loop["times"], D, std=0.3)
    for i, l in enumerate(cfg["layers"]):
        p, m, x = f"l{i}.", l["mixer"], f"l{i}.mix."
        sd[p + "norm1"] = rn(D, std=0.2)
        if l["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            sd[x + "q"], sd[x + "k"], sd[x + "v"] = lin(H * dk, D), lin(G * dk, D), lin(G * dv, D)
            sd[x + "q.norm"], sd[x + "k.norm"] = 1 + rn(H * dk, std=0.3), 1 + rn(G * dk, std=0.3)
            sd[x + "r1"], sd[x + "r2"] = un(H, lo=0.2, hi=1.5), un(H, lo=0.1, hi=2.0)
            sd[x + "g"], sd[x + "o"] = lin(H * dv, D), lin(D, H * dv)
        elif l["type"] == "wkv":
            H, d = m["heads"], m["dim"]
            r = 6
            for s in "rkvgw":
                sd[x + "mu." + s] = un(D)
            for s in "rkvg":
                sd[x + s] = lin(H * d, D)
            sd[x + "w1"], sd[x + "w2"] = lin(r, D), lin(H * d, r)
            sd[x + "w0"] = un(H * d, lo=-7.0, hi=-5.0) if slow_decay else un(H * d, lo=-3.0, hi=0.5)
            sd[x + "u"] = rn(H, d, std=0.5)
            sd[x + "norm"] = 1 + rn(H * d, std=0.2)
            sd[x + "o"] = lin(D, H * d)
        else:
            H, G, dk, dv, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            r = 5
            for s, n in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
                sd[x + s] = lin(n, D)
                sd[x + s + ".conv"] = rn(n, K, std=0.7)
            sd[x + "b"] = lin(H, D)
            sd[x + "A_log"] = torch.log(un(H, lo=0.5, hi=3.0)).to(torch.bfloat16).float()
            sd[x + "norm"] = 1 + rn(dv, std=0.2)
            sd[x + "a1"], sd[x + "a2"] = lin(r, D), lin(H * dk, r)
            sd[x + "dt_bias"] = un(H * dk, lo=-8.0, hi=-6.0) if slow_decay else un(H * dk, lo=-3.0, hi=0.5)
            sd[x + "g1"], sd[x + "g2"] = lin(r, D), lin(H * dv, r)
            sd[x + "o"] = lin(D, H * dv)
        if l.get("mlp") is not None:
            ff = l["mlp"]["ff"]
            sd[p + "norm2"] = rn(D, std=0.2)
            sd[p + "mlp.up"], sd[p + "mlp.down"] = lin(ff, D), lin(D, ff)
            sd[p + "mlp.act"] = torch.tensor([0.7, 0.4, 0.25, 0.1]) + rn(4, std=0.05)
    return {k: v.to(torch.bfloat16).float() for k, v in sd.items()}  # every value survives a bf16 checkpoint


def make_config(layers, width=48, vocab=96, loop=None, eps=1e-5, mult=0.5, scale=6.0) -> dict:
    cfg = {"architecture": "Pinavik", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
           "residual_mult": mult, "embedding": {"scale": scale}}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def att(dim=16, vdim=16, heads=4, kv_heads=2, window=6, scale=0.3, softcap=4.0):
    return {"type": "attention", "mixer": {"dim": dim, "vdim": vdim, "heads": heads, "kv_heads": kv_heads,
                                           "mask": {"size": window}, "scale": scale, "softcap": softcap}}


def wkv(dim=8, heads=3):
    return {"type": "wkv", "mixer": {"dim": dim, "heads": heads}}


def cdelta(dim=8, vdim=12, heads=4, kv_heads=2, conv=4):
    return {"type": "channel_delta", "mixer": {"dim": dim, "vdim": vdim, "heads": heads, "kv_heads": kv_heads,
                                               "conv": conv}}


def with_mlp(layer, ff=64):
    return dict(layer, mlp=None if ff is None else {"kind": "dense", "ff": ff})

"""Slow float64 oracle of the Ronavik decoder, written from its equations: one function per mechanism, whole sequences
at once, plain loops for the recurrences. It shares no code with the framework (no ops, no engine, no model class); it
reads the checkpoint layout (tensor names) and the config dictionary only.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms_div(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(x, w, b):
    """x [T, C], w [C, taps] (last column = the current token), zeros before the start."""
    T, C = x.shape
    K = w.shape[1]
    pad = torch.cat([torch.zeros(K - 1, C, dtype=F64), x])
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for i in range(K):
            y[t] += pad[t + i] * w[:, i]
    return y + b


def sigmoid_attention(h, W, p, m, eps):
    """Causal attention whose key weights are sigmoid(score + bias_h), not normalised over the keys."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = norm((h @ W[p + "q"].T).reshape(T, H, dk), W[p + "q.norm"], eps)
    k = norm((h @ W[p + "k"].T).reshape(T, G, dk), W[p + "k.norm"], eps)
    v = (h @ W[p + "v"].T).reshape(T, G, dv)
    qt = m.get("q_temp")
    heads = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        temp = 1.0
        if qt:
            temp = 1.0 + qt["coef"] * math.log((i + 1) // qt["every"] + 1)
        for hh in range(H):
            g = hh // (H // G)
            for j in range(i + 1):
                s = float((q[i, hh] * temp) @ k[j, g]) * m["scale"]
                heads[i, hh] += v[j, g] / (1.0 + math.exp(-(s + float(W[p + "pb"][hh]))))
    return heads.reshape(T, H * dv) @ W[p + "o"].T


def gated_linear_recurrence(h, W, p, m):
    """Recurrent block: a gelu branch times a real-gated linear recurrent unit over a short convolution."""
    T = h.shape[0]
    Wd, nb = m["width"], m["blocks"]
    y = gelu_tanh(h @ W[p + "y"].T + W[p + "y.b"])
    u = causal_conv(h @ W[p + "x"].T + W[p + "x.b"], W[p + "conv"], W[p + "conv.b"])
    bs = Wd // nb
    r = torch.zeros(T, Wd, dtype=F64)
    ig = torch.zeros(T, Wd, dtype=F64)
    for b in range(nb):
        ub = u[:, b * bs:(b + 1) * bs]
        r[:, b * bs:(b + 1) * bs] = torch.sigmoid(ub @ W[p + "ra"][b].T + W[p + "ra.b"][b])
        ig[:, b * bs:(b + 1) * bs] = torch.sigmoid(ub @ W[p + "ri"][b].T + W[p + "ri.b"][b])
    log_a = -8.0 * r * torch.nn.functional.softplus(W[p + "lam"])
    a = torch.exp(log_a)
    S = torch.zeros(Wd, dtype=F64)
    out = torch.zeros(T, Wd, dtype=F64)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * ig[t] * u[t]
        out[t] = S * y[t]
    return out @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    left = sigmoid_attention(h, W, p + "left.", m["left"], eps)
    right = gated_linear_recurrence(h, W, p + "right.", m["right"])
    return m.get("left_scale", 1.0) * left + m.get("right_scale", 1.0) * right


def mamba2_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * dv
    proj = h @ W[p + "in"].T
    z = proj[:, :inner]
    xbc = proj[:, inner:2 * inner + 2 * G * N]
    dt = proj[:, 2 * inner + 2 * G * N:]
    xbc = torch.nn.functional.silu(causal_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, dv)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = torch.nn.functional.softplus(dt + W[p + "dt_bias"])
    y = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(N, dv, dtype=F64)
        A = math.exp(float(W[p + "A_log"][hh]))
        for t in range(T):
            S = math.exp(-A * float(dt[t, hh])) * S + float(dt[t, hh]) * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S.T @ C[t, g] + W[p + "D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * torch.nn.functional.silu(z)
    ng = m.get("norm_groups", 1)
    y = rms_div(y.reshape(T, ng, inner // ng), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def moe(h, W, p, ml, gaps=None):
    """Sigmoid router; the chosen experts' scores scale each expert's INPUT; experts are W_down relu(W_up .)^2."""
    T = h.shape[0]
    E, top = ml["router"]["experts"], ml["router"]["top"]
    s = torch.sigmoid(h @ W[p + "router"].T)
    if gaps is not None and top < E:
        ss = s.sort(-1, descending=True).values
        gaps.append(float((ss[:, top - 1] - ss[:, top]).min()))
    out = torch.zeros(T, W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            a = torch.relu(W[p + f"e{e}.up"] @ (s[t, e] * h[t])) ** 2
            out[t] += W[p + f"e{e}.down"] @ a
    return out


def forward(cfg: dict, W: dict, tokens, residuals: list | None = None, gaps: list | None = None):
    """tokens: list of ints -> logits [T, vocab] (float64). `residuals` collects the stream after every layer."""
    W = {k: v.to(F64) if v.is_floating_point() else v for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    x = W["embed"][torch.tensor(tokens)] + W["pos"][:T]
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = norm(x, W[p + "norm1"], eps)
        if l["type"] == "parallel":
            y = parallel_mixer(h, W, p + "mix.", l["mixer"], eps)
        elif l["type"] == "mamba2":
            y = mamba2_mixer(h, W, p + "mix.", l["mixer"], eps)
        else:
            raise ValueError(l["type"])
        y = y * torch.sigmoid(h @ W[p + "rg1"].T + W[p + "rg1.b"])
        x = x + norm(y, W[p + "norm1b"], eps)
        if l.get("mlp") is not None:
            h = norm(x, W[p + "norm2"], eps)
            y = moe(h, W, p + "mlp.", l["mlp"], gaps)
            y = y * torch.sigmoid(h @ W[p + "rg2"].T + W[p + "rg2.b"])
            x = x + norm(y, W[p + "norm2b"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    return norm(x, W["final.norm"], eps) @ W["embed"].T


# ------------------------------------------------------------------------------------------------ test model builders
def par(dim=8, vdim=12, heads=4, kv_heads=2, scale=0.35, q_temp=(0.5, 4), width=24, blocks=3, conv=3, left_scale=0.7,
        right_scale=1.4):
    left = dict(dim=dim, vdim=vdim, heads=heads, kv_heads=kv_heads, scale=scale)
    if q_temp:
        left["q_temp"] = dict(coef=q_temp[0], every=q_temp[1])
    return dict(type="parallel", mixer=dict(left=left, right=dict(width=width, blocks=blocks, conv=conv),
                                            left_scale=left_scale, right_scale=right_scale))


def ssm(heads=4, vdim=8, state=12, groups=2, norm_groups=4, conv=4):
    return dict(type="mamba2", mixer=dict(heads=heads, vdim=vdim, state=state, groups=groups, norm_groups=norm_groups,
                                          conv=conv))


def with_mlp(layer, ff=24, experts=5, top=2):
    mlp = None if ff is None else dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))
    return dict(layer, mlp=mlp)


def make_config(layers, width=32, vocab=97, eps=1e-5, max_positions=400):
    return dict(architecture="Ronavik", vocab=vocab, width=width, max_positions=max_positions, norm=dict(eps=eps),
                layers=list(layers))


def random_checkpoint(cfg, seed, slow_decay=False):
    """Random weights under the checkpoint's tensor names, rounded to bfloat16 (what a stored checkpoint holds), with
    magnitudes that make every mechanism matter: sizeable position vectors, biases, gate matrices and routers."""
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]

    def rn(*s, std=1.0):
        return (torch.randn(*s, generator=g) * std).to(torch.bfloat16).float()

    def un(*s, lo=0.0, hi=1.0):
        return (torch.rand(*s, generator=g) * (hi - lo) + lo).to(torch.bfloat16).float()

    def lin(o, i, gain=1.0):
        return rn(o, i, std=gain * i ** -0.5)

    W = {"embed": rn(cfg["vocab"], D), "pos": rn(cfg["max_positions"], D, std=0.5), "final.norm": un(D, lo=0.5, hi=1.5)}
    for i, l in enumerate(cfg["layers"]):
        p, x, m = f"l{i}.", f"l{i}.mix.", l["mixer"]
        W[p + "norm1"], W[p + "norm1b"] = un(D, lo=0.5, hi=1.5), un(D, lo=0.5, hi=1.5)
        W[p + "rg1"], W[p + "rg1.b"] = lin(D, D, 2.0), rn(D)
        if l["type"] == "parallel":
            a, r = m["left"], m["right"]
            H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            xl, xr = x + "left.", x + "right."
            W[xl + "q"], W[xl + "k"], W[xl + "v"] = lin(H * dk, D, 2.0), lin(G * dk, D, 2.0), lin(G * dv, D)
            W[xl + "q.norm"], W[xl + "k.norm"] = un(dk, lo=0.5, hi=1.5), un(dk, lo=0.5, hi=1.5)
            W[xl + "pb"] = un(H, lo=-3.0, hi=0.0)
            W[xl + "o"] = lin(D, H * dv)
            Wd, nb, K = r["width"], r["blocks"], r["conv"]
            bs = Wd // nb
            W[xr + "y"], W[xr + "y.b"] = lin(Wd, D), rn(Wd, std=0.3)
            W[xr + "x"], W[xr + "x.b"] = lin(Wd, D), rn(Wd, std=0.3)
            W[xr + "conv"], W[xr + "conv.b"] = rn(Wd, K, std=0.6), rn(Wd, std=0.2)
            W[xr + "ra"], W[xr + "ra.b"] = rn(nb, bs, bs, std=2.0 * bs ** -0.5), rn(nb, bs)
            W[xr + "ri"], W[xr + "ri.b"] = rn(nb, bs, bs, std=2.0 * bs ** -0.5), rn(nb, bs)
            W[xr + "lam"] = un(Wd, lo=-9.0, hi=-6.0) if slow_decay else un(Wd, lo=-4.0, hi=0.5)
            W[xr + "o"] = lin(D, Wd)
        else:
            H, dv, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            inner, C = H * dv, H * dv + 2 * G * N
            W[x + "in"] = lin(2 * inner + 2 * G * N + H, D, 1.5)
            W[x + "conv"], W[x + "conv.b"] = rn(C, K, std=0.6), rn(C, std=0.2)
            W[x + "dt_bias"] = un(H, lo=-6.0, hi=-4.0) if slow_decay else un(H, lo=-2.0, hi=1.0)
            W[x + "A_log"] = un(H, lo=-2.0, hi=-1.0) if slow_decay else un(H, lo=-1.0, hi=1.2)
            W[x + "D"] = rn(H)
            W[x + "norm"] = un(inner, lo=0.5, hi=1.5)
            W[x + "o"] = lin(D, inner)
        ml = l.get("mlp")
        if ml is not None:
            F_, E = ml["expert"]["ff"], ml["router"]["experts"]
            W[p + "norm2"], W[p + "norm2b"] = un(D, lo=0.5, hi=1.5), un(D, lo=0.5, hi=1.5)
            W[p + "rg2"], W[p + "rg2.b"] = lin(D, D, 2.0), rn(D)
            W[p + "mlp.router"] = lin(E, D, 3.0)
            for e in range(E):
                W[p + f"mlp.e{e}.up"], W[p + f"mlp.e{e}.down"] = lin(F_, D, 1.5), lin(D, F_)
    return W


def router_margin(cfg, W, tokens):
    """Smallest gap between the last chosen and the first not chosen router score over all layers and positions (a test
    with a near-tie would rest on rounding)."""
    gaps = []
    forward(cfg, W, tokens, gaps=gaps)
    return min(gaps) if gaps else 1.0

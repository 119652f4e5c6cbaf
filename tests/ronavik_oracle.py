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


def moe(h, W, p, ml):
    """Sigmoid router; the chosen experts' scores scale each expert's INPUT; experts are W_down relu(W_up .)^2."""
    T = h.shape[0]
    E, top = ml["router"]["experts"], ml["router"]["top"]
    s = torch.sigmoid(h @ W[p + "router"].T)
    out = torch.zeros(T, W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            a = torch.relu(W[p + f"e{e}.up"] @ (s[t, e] * h[t])) ** 2
            out[t] += W[p + f"e{e}.down"] @ a
    return out


def forward(cfg: dict, W: dict, tokens, residuals: list | None = None):
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
            y = moe(h, W, p + "mlp.", l["mlp"])
            y = y * torch.sigmoid(h @ W[p + "rg2"].T + W[p + "rg2.b"])
            x = x + norm(y, W[p + "norm2b"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    return norm(x, W["final.norm"], eps) @ W["embed"].T

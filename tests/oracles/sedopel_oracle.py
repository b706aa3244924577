"""Slow float64 oracle of the Sedopel design, one function per mechanism, written from the design's
equations and sharing no code with the product path.

Notation: h is a sublayer's input [T, width]; positions count from 0;
rms(x) = x / sqrt(mean(x^2) + eps).  Weights come as a dict under the checkpoint's names
('l<i>.mix.<name>', 'l<i>.mlp.<name>'), the configuration as the parsed config.json.
"""
import math

import torch

F64 = torch.float64


def rms(x, eps, w=None):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def gelu_erf(x):
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def rotate_half(x, pos, dims, base):
    """Rotate the first ``dims`` entries of the last axis of x [T, heads, d]; entry i pairs with
    i + dims/2; angle = position * base^(-2i/dims)."""
    half = dims // 2
    if half == 0:
        return x
    f = base ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    a = pos.to(F64)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half], out[..., half:dims] = u * c - v * s, v * c + u * s
    return out


def short_conv(x, w):
    """Causal convolution per channel, zeros before the start: x [T, C], w [C, taps] whose last
    column multiplies the current token."""
    T, C = x.shape
    K = w.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=F64), x], 0)
    return torch.stack([(padded[t:t + K] * w.T).sum(0) for t in range(T)])


def softmax_attention(h, W, p, m, eps):
    """Grouped-query causal softmax attention: rotation on part of each head, then unit-RMS q and k,
    scores times scale times a per-head temperature, a sigmoid gate on the concatenated heads."""
    T, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ W[p + "q"].T).view(T, H, d)
    k = (h @ W[p + "k"].T).view(T, G, d)
    v = (h @ W[p + "v"].T).view(T, G, dv)
    rot = m.get("rot")
    if rot:
        q, k = rotate_half(q, pos, rot["dims"], rot["base"]), rotate_half(k, pos, rot["dims"], rot["base"])
    q, k = rms(q, eps), rms(k, eps)
    out = torch.zeros(T, H, dv, dtype=F64)
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * m["scale"] * W[p + "temp"][hh]
        s = s.masked_fill(~mask, float("-inf"))
        out[:, hh] = torch.softmax(s, -1) @ v[:, g]
    o = out.reshape(T, H * dv) * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def lightning(h, W, p, m, eps):
    """Linear attention with a fixed decay per head: S <- decay S + k v^T, o = S^T q over SiLU'd
    projections; the heads are normed together, gated by a sigmoid, projected."""
    T, H, d, dv = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].T).view(T, H, d)
    k = silu(h @ W[p + "k"].T).view(T, H, d)
    v = silu(h @ W[p + "v"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            S = m["decay"][hh] * S + torch.outer(k[t, hh], v[t, hh])
            out[t, hh] = S.T @ q[t, hh]
    o = rms(out.reshape(T, H * dv), eps, W[p + "norm"]) * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def parallel(h, W, p, m, eps):
    """Two mixers over the same input; each output is RMS-normed over the width with its own
    weight, the result is half their sum."""
    a = rms(softmax_attention(h, W, p + "left.", m["left"], eps), eps, W[p + "left.out"])
    b = rms(lightning(h, W, p + "right.", m["right"], eps), eps, W[p + "right.out"])
    return 0.5 * (a + b)


def delta(h, W, p, m, eps):
    """Gated delta rule: per head S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(T, G, d)
    k = silu(short_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(T, G, d)
    v = silu(short_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(T, H, dv)
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q, k = unit(q) * d ** -0.5, unit(k)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    g = torch.exp(-torch.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        kv = hh // (H // G)
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            S = g[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            out[t, hh] = S.T @ q[t, kv]
    o = rms(out, eps, W[p + "norm"]).reshape(T, H * dv) * silu(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def dense_ff(h, W, p):
    return gelu_erf(h @ W[p + "up"].T) @ W[p + "down"].T


def forward(cfg, weights, tokens, taps=None):
    """Logits [T, vocab] of one sequence; ``taps`` collects the stream after every layer."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    outs = [x]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms(x, eps, W[p + "norm1"])
        y = parallel(h, W, p + "mix.", L["mixer"], eps) if L["type"] == "parallel" else delta(h, W, p + "mix.", L["mixer"], eps)
        x = x + rms(y, eps, W[p + "norm1b"])
        if L.get("mlp"):
            x = x + rms(dense_ff(rms(x, eps, W[p + "norm2"]), W, p + "mlp."), eps, W[p + "norm2b"])
        outs.append(x)
        x = sum(W[p + "dwa"][j] * outs[j] for j in range(i + 2))
        if taps is not None:
            taps.append(x)
    return rms(x, eps, W["final.norm"]) @ W["head"].T


def greedy(cfg, weights, prompt, n):
    """n arg-max continuations of a prompt (the whole sequence is recomputed every step)."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(cfg, weights, toks)[-1])))
    return toks[len(prompt):]

"""Slow float64 oracle of the Filevik design, one function per mechanism, written from the
design's equations and sharing no code with the product path.

Notation: h is a sublayer's input [T, width]; positions count from 0; rms(x) = x / sqrt(mean(x^2) + eps).
Weights come as a dict under the checkpoint's names ('l<i>.mix.<name>', 'l<i>.mlp.<name>').
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


def rotate(x, pos, dims, base, interleaved):
    """Rotate the first ``dims`` entries of the last axis of x [T, heads, d]: pair i is (i, i + dims/2)
    ('half') or (2i, 2i + 1) (interleaved); angle = position * base^(-2i/dims)."""
    half = dims // 2
    if half == 0:
        return x
    f = base ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    a = pos.to(F64)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2], out[..., 1:dims:2] = u * c - v * s, v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half], out[..., half:dims] = u * c - v * s, v * c + u * s
    return out


def mamba1(h, W, p, m):
    """x, z = split(W_in h); x = silu(causal conv(x)); dt, B, C = split(W_x x);
    dt = softplus(W_dt dt + b); S <- exp(dt A) S + dt x B; y = S C + D x; out = W_o (y silu(z))."""
    T, C, N, R, K = h.shape[0], m["inner"], m["state"], m["dt_rank"], m["conv"]
    xz = h @ W[p + "in"].T
    x, z = xz[:, :C], xz[:, C:]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=F64), x], 0)
    conv = torch.stack([(padded[t:t + K] * W[p + "conv"].T).sum(0) for t in range(T)]) + W[p + "conv.b"]
    x = silu(conv)
    proj = x @ W[p + "x"].T
    dt = softplus(proj[:, :R] @ W[p + "dt"].T + W[p + "dt.b"])
    Bm, Cm = proj[:, R:R + N], proj[:, R + N:R + 2 * N]
    A = -torch.exp(W[p + "A_log"])
    S = torch.zeros(C, N, dtype=F64)
    ys = []
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * Bm[t][None, :]
        ys.append(S @ Cm[t] + W[p + "D"] * x[t])
    return (torch.stack(ys) * silu(z)) @ W[p + "o"].T


def retention(h, W, p, m, eps):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t; heads to unit RMS, times silu(W_g h), W_o."""
    T, H, d, dv = h.shape[0], m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate((h @ W[p + "q"].T).view(T, H, d), pos, rot["dims"], rot["base"], False)
    k = rotate((h @ W[p + "k"].T).view(T, H, d), pos, rot["dims"], rot["base"], False) * d ** -0.5
    v = (h @ W[p + "v"].T).view(T, H, dv)
    dec = torch.tensor(m["decay"], dtype=F64)
    S = torch.zeros(H, d, dv, dtype=F64)
    os_ = []
    for t in range(T):
        S = dec[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        os_.append(torch.einsum("hdv,hd->hv", S, q[t]))
    o = rms(torch.stack(os_), eps).reshape(T, H * dv) * silu(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def latent_attention(h, W, p, m, eps):
    """Queries through a normed latent; keys and values from a normed shared latent c plus one rotated
    key part shared by the heads; causal softmax of (q_n . k_n + q_r . k_r) * scale."""
    T, H, d, dr, dv, r = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (rms(h @ W[p + "dq"].T, eps, W[p + "dq.norm"]) @ W[p + "uq"].T).view(T, H, d + dr)
    down = h @ W[p + "dkv"].T
    c = rms(down[:, :r], eps, W[p + "dkv.norm"])
    rot = m["rot"]
    qr = rotate(q[..., d:], pos, rot["dims"], rot["base"], True)
    kr = rotate(down[:, r:].view(T, 1, dr), pos, rot["dims"], rot["base"], True)[:, 0]
    kn = (c @ W[p + "uk"].T).view(T, H, d)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    sc = (torch.einsum("thd,shd->hts", q[..., :d], kn) + torch.einsum("thd,sd->hts", qr, kr)) * m["scale"]
    sc = sc.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), -math.inf)
    o = torch.einsum("hts,shv->thv", torch.softmax(sc, -1), v).reshape(T, H * dv)
    return o @ W[p + "o"].T


def experts(h, W, p, f):
    """softmax router over all experts, the ``top`` largest renormalised (+1e-20) and scaled; expert =
    W_down relu(W_up h)^2; plus the shared expert."""
    ro = f["router"]
    s = torch.softmax(h @ W[p + "router"].T, -1)
    val, idx = torch.topk(s, ro["top"], -1)
    w = val / (val.sum(-1, keepdim=True) + 1e-20) * ro.get("scale", 1.0)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ro["top"]):
            e = int(idx[t, j])
            out[t] += w[t, j] * ((torch.relu(h[t] @ W[p + f"e{e}.up"].T) ** 2) @ W[p + f"e{e}.down"].T)
    if f.get("shared"):
        out = out + (torch.relu(h @ W[p + "shared.up"].T) ** 2) @ W[p + "shared.down"].T
    return out


def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` collects the residual stream per layer."""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(list(tokens))]
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        if L["type"] == "mamba1":
            y = mamba1(x, W, p, m)
        elif L["type"] == "retention":
            y = retention(x, W, p, m, eps)
        elif L["type"] == "latent_attention":
            y = latent_attention(x, W, p, m, eps)
        else:
            raise ValueError(L["type"])
        x = x + rms(y, eps, W[f"l{i}.norm1"])
        if L.get("mlp"):
            x = x + rms(experts(x, W, f"l{i}.mlp.", L["mlp"]), eps, W[f"l{i}.norm2"])
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rms(x, eps, W["final.norm"]) @ W["head"].T) * cfg.get("logit_scale", 1.0)


def greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]

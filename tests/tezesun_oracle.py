"""A plain, slow float64 model of the Tezesun design, written from its equations: one function per mechanism, a
whole-sequence forward pass over them. It shares no code with the package; the tests compare the package with it.

A Tezesun layer reads ONE RMS norm of the residual stream x: with h = rms(x) w,

    x <- x + ls1 * mixer(shifted(h)) + ls2 * ff(h)

`shifted` blends every token's h with the previous token's h (zeros before the first) by a learned vector. The
mixer is a real-gated linear recurrent unit (`rglru`), differential attention over a sliding window that also keeps
the sequence's first tokens (`attention`), or attention through a low-rank latent (`latent_attention`); the
feed-forward is up -> xIELU -> down.
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def softplus(x):
    return torch.log1p(torch.exp(-x.abs())) + x.clamp(min=0)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z / 2; z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2."""
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (torch.expm1(z.clamp(max=0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def token_shift(h, mu):
    """h [T, W] of one whole sequence -> h + (previous h - h) * mu, the previous of token 0 being zeros."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (prev - h) * mu


def causal_conv(x, taps, bias):
    """x [T, C], taps [C, K] (last column on the current token), zeros before the start."""
    T, K = x.shape[0], taps.shape[1]
    pad = torch.cat([torch.zeros(K - 1, x.shape[1], dtype=x.dtype), x])
    return sum(pad[j:j + T] * taps[:, j] for j in range(K)) + bias


def rglru(h, w):
    """y = gelu(W_y h + b), u = conv(W_x h + b); per block gates r, i = sigmoid(block matrix u_b + b);
    a = exp(-8 r softplus(lam)); S <- a S + sqrt(1 - a^2) i u; out = W_o (S * y)."""
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    u = causal_conv(h @ w["x"].T + w["x.b"], w["conv"], w["conv.b"])
    nb, bw = w["ra"].shape[0], w["ra"].shape[1]
    ub = u.reshape(-1, nb, bw)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w["ra"]) + w["ra.b"]).reshape(u.shape)
    i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w["ri"]) + w["ri.b"]).reshape(u.shape)
    a = torch.exp(-8.0 * r * softplus(w["lam"]))
    S = torch.zeros(u.shape[1], dtype=F64)
    out = []
    for t in range(u.shape[0]):
        S = a[t] * S + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        out.append(S * y[t])
    return torch.stack(out) @ w["o"].T


def rope_angles(rot, T):
    """(cos, sin) [T, dims / 2] for positions 0 .. T-1: frequencies base^(-2i / dims), optionally rescaled
    (a ramp between two wavelengths picks per frequency between f and f / factor; cos and sin grow by 0.1 ln(factor) + 1)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    mult = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])
        turn = lambda t: dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))
        lo = max(math.floor(turn(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn(float(sc["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mult = 0.1 * math.log(factor) + 1.0
    ang = torch.arange(T, dtype=F64).unsqueeze(1) * f
    return torch.cos(ang) * mult, torch.sin(ang) * mult


def rotate(x, cos, sin, interleaved):
    """x [T, n, D]: the first 2 * cos.shape[1] entries of every vector are rotated, pairs (2i, 2i + 1) when
    `interleaved`, else (i, i + dims / 2); the rest pass."""
    half = cos.shape[1]
    dims = 2 * half
    head, tail = x[..., :dims], x[..., dims:]
    c, s = cos.unsqueeze(1), sin.unsqueeze(1)
    if interleaved:
        u, v = head[..., 0::2], head[..., 1::2]
        out = torch.stack([u * c - v * s, v * c + u * s], dim=-1).reshape(head.shape)
    else:
        u, v = head[..., :half], head[..., half:]
        out = torch.cat([u * c - v * s, v * c + u * s], dim=-1)
    return torch.cat([out, tail], dim=-1)


def visible(T, size, keep_first):
    i = torch.arange(T).unsqueeze(1)
    j = torch.arange(T).unsqueeze(0)
    ok = j <= i
    if size:
        ok = ok & ((i - j < size) | (j < keep_first))
    return ok


def diff_attention(h, w, m, eps):
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w["q"].T).reshape(T, H * 2, d)
    k = (h @ w["k"].T).reshape(T, G * 2, d)
    v = (h @ w["v"].T).reshape(T, G, dv)
    if m.get("rot"):
        cos, sin = rope_angles(m["rot"], T)
        q, k = rotate(q, cos, sin, True), rotate(k, cos, sin, True)
    mask = m.get("mask") or {}
    ok = visible(T, int(mask.get("size") or 0), int(mask.get("keep_first") or 0))
    diff = float(m["diff"])
    lam = torch.exp((w["lq1"] * w["lk1"]).sum()) - torch.exp((w["lq2"] * w["lk2"]).sum()) + diff
    cap = float(m.get("softcap") or 0.0)
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        maps = []
        for mp in range(2):
            s = (q[:, 2 * hh + mp] @ k[:, 2 * g + mp].T) * float(m["scale"])
            if cap > 0:
                s = cap * torch.tanh(s / cap)
            s = s.masked_fill(~ok, float("-inf"))
            maps.append(torch.softmax(s, dim=-1) @ v[:, g])
        o = maps[0] - lam * maps[1]
        heads.append(rms(o, eps) * (1.0 - diff))
    o = torch.cat(heads, dim=-1) * torch.sigmoid(h @ w["g"].T)
    return o @ w["o"].T


def latent_attention(h, w, m, eps):
    T = h.shape[0]
    H, d, dr, dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    cq = rms(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).reshape(T, H, d + dr)
    kv = h @ w["dkv"].T
    c = rms(kv[:, :R], eps) * w["dkv.norm"]
    cos, sin = rope_angles(m["rot"], T)
    kr = rotate(kv[:, R:].reshape(T, 1, dr), cos, sin, False)[:, 0]
    qr = rotate(q[..., d:], cos, sin, False)
    ku = (c @ w["uk"].T).reshape(T, H, d)
    v = (c @ w["uv"].T).reshape(T, H, dv)
    ok = visible(T, 0, 0)
    heads = []
    for hh in range(H):
        s = (q[:, hh, :d] @ ku[:, hh].T + qr[:, hh] @ kr.T) * float(m["scale"])
        s = s.masked_fill(~ok, float("-inf"))
        heads.append(torch.softmax(s, dim=-1) @ v[:, hh])
    return torch.cat(heads, dim=-1) @ w["o"].T


def feed_forward(h, w):
    return xielu(h @ w["up"].T, w["act"][0], w["act"][1]) @ w["down"].T


def forward(cfg, sd, tokens):
    """cfg: the config.json dict, sd: name -> tensor, tokens: one whole sequence.
    Returns (logits [T, vocab], the residual stream after every layer [layers, T, width]) in float64."""
    t = {k: v.to(F64) for k, v in sd.items()}
    eps = float(cfg["norm"]["eps"])
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        w = {k[len(p) + 4:]: v for k, v in t.items() if k.startswith(p + "mix.")}
        h = rms(x, eps) * t[p + "norm1"]
        hs = token_shift(h, t[p + "shift"])
        m = layer["mixer"]
        if layer["type"] == "rglru":
            y = rglru(hs, w)
        elif layer["type"] == "attention":
            y = diff_attention(hs, w, m, eps)
        elif layer["type"] == "latent_attention":
            y = latent_attention(hs, w, m, eps)
        else:
            raise ValueError(layer["type"])
        add = y * t[p + "ls1"]
        if layer.get("mlp") is not None:
            f = {k[len(p) + 4:]: v for k, v in t.items() if k.startswith(p + "mlp.")}
            add = add + feed_forward(h, f) * t[p + "ls2"]
        x = x + add
        after.append(x)
    logits = (rms(x, eps) * t["final.norm"]) @ t["head"].T * float(cfg.get("logit_scale", 1.0))
    return logits, torch.stack(after)

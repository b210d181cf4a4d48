"""A plain, slow model of the Zovozen design in float64, one function per mechanism, written from the design's equations.
It shares no code with the package: it parses the config dictionary itself, takes the checkpoint's tensors by name, and
runs ONE whole sequence at a time (no cache, no batching), so everything the engine does with caches, slots and steps
can be held against it.

A layer:  x <- x + norm1(mixer(x));  x <- x + norm2(ff(x))   (the sublayers read x itself; RMS norms with weights).
The mixer is a pair reading the same input: attention ("left") beside a matrix memory ("right"),
left_scale * left + right_scale * right.
"""
import math

import torch

F64 = torch.float64


def rms(x, eps, w=None):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_half_partial(x, pos, dims, base, factor):
    """x [T, heads, D]; the first `dims` entries of every vector are rotated, entry i paired with i + dims / 2, by the
    angle pos * base^(-2i / dims) / factor."""
    if not dims:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=F64)
    a = pos.to(F64).view(-1, 1, 1) * f.view(1, 1, half)
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def chunk_mask(T, size, pos0=0):
    """visible[i, j]: j <= i and both in the same chunk of `size` positions (size 0: plain causal)."""
    p = torch.arange(pos0, pos0 + T)
    vis = p.view(1, -1) <= p.view(-1, 1)
    if size:
        vis = vis & ((p.view(1, -1) // size) == (p.view(-1, 1) // size))
    return vis


def mixed_scores(q, k, scale, temp, talk):
    """q [T, H, d], k [T, G, d] -> [H, T, T]: (q . k) * scale * temp[h], then the heads' scores mixed by talk [H, H]."""
    H, G = q.shape[1], k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale * temp.view(H, 1, 1)
    return torch.einsum("hg,gij->hij", talk, s)


def sink_softmax(s, vis, sink):
    """softmax over the visible keys with one more term exp(sink[h]) in the denominator."""
    s = s.masked_fill(~vis.unsqueeze(0), float("-inf"))
    m = torch.maximum(s.max(-1, keepdim=True).values, sink.view(-1, 1, 1))
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink.view(-1, 1, 1) - m))


def left_attention(h, P, c, eps):
    """P: the tensors under '<layer>.mix.left.' by short name; c: the config's mixer.left."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = h @ P["q"].T + P["q.b"]
    k = h @ P["k"].T + P["k.b"]
    v = h @ P["v"].T + P["v.b"]
    q = rms(q, eps, P["q.norm"]).view(T, H, d)          # over the whole projection, before the split into heads
    k = rms(k, eps, P["k.norm"]).view(T, G, d)
    rot = c.get("rot") or {}
    pos = torch.arange(T)
    factor = float(((rot.get("scaling") or {}).get("factor")) or 1.0)
    q = rotate_half_partial(q, pos, int(rot.get("dims", 0)), float(rot.get("base", 1.0)), factor)
    k = rotate_half_partial(k, pos, int(rot.get("dims", 0)), float(rot.get("base", 1.0)), factor)
    v = rms(v.view(T, G, dv), eps)
    s = mixed_scores(q, k, c["scale"], P["temp"], P["talk"])
    p = sink_softmax(s, chunk_mask(T, int((c.get("mask") or {}).get("size") or 0)), P["sink"])
    o = torch.einsum("hij,jhd->ihd", p, v.repeat_interleave(H // G, dim=1)).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ P["g"].T)
    return o @ P["o"].T + P["o.b"]


def matrix_memory(q, k, v, li, lf):
    """q, k [T, H, d], v [T, H, dv], log gates [T, H]. S, n, m start at zero (m at 0, not at minus infinity)."""
    T, H, d = q.shape
    dv = v.shape[2]
    S, n, m = torch.zeros(H, d, dv, dtype=F64), torch.zeros(H, d, dtype=F64), torch.zeros(H, dtype=F64)
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(lf[t] + m, li[t])
        a, b = torch.exp(lf[t] + m - m_new), torch.exp(li[t] - m_new)
        S = a.view(H, 1, 1) * S + b.view(H, 1, 1) * k[t].unsqueeze(2) * v[t].unsqueeze(1)
        n = a.view(H, 1) * n + b.view(H, 1) * k[t]
        m = m_new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = torch.einsum("hdv,hd->hv", S, q[t]) / den.view(H, 1)
    return out


def right_memory(h, P, c, eps):
    T = h.shape[0]
    H, d, dv, cap = c["heads"], c["dim"], c["vdim"], float(c["gate_cap"])
    q = (h @ P["q"].T).view(T, H, d) * d ** -0.5
    k = (h @ P["k"].T).view(T, H, d)
    v = (h @ P["v"].T).view(T, H, dv)
    li = cap * torch.tanh((h @ P["i"].T + P["i.b"]) / cap)
    lf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ P["f"].T + P["f.b"]) / cap))
    o = rms(matrix_memory(q, k, v, li, lf), eps).reshape(T, H * dv)
    return (o * P["norm"] * torch.sigmoid(h @ P["g"].T)) @ P["o"].T


def dense_ff(h, P):
    z = torch.relu(h @ P["up"].T + P["up.b"])
    return (z * z) @ P["down"].T + P["down.b"]


def gated_expert(h, P, pre):
    g = h @ P[pre + "gate"].T
    return (g * torch.sigmoid(g) * (h @ P[pre + "up"].T)) @ P[pre + "down"].T


def route(h, P, r):
    """-> (chosen [T, top], weights [T, top]). Softmax scores over all router outputs; the choice goes by score + correction
    within the best `keep` groups (a group's rank: its largest choice score), the weights are the plain scores."""
    E, top = P["router"].shape[0], int(r["top"])
    g = r.get("groups") or {}
    ng, keep = int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))
    s = torch.softmax(h @ P["router"].T, dim=-1)
    choice = s + P["correction"]
    T = h.shape[0]
    per = E // ng
    gs = choice.view(T, ng, per).max(-1).values
    kept = torch.zeros(T, ng, dtype=torch.bool)
    kept.scatter_(1, torch.argsort(gs, dim=-1, descending=True, stable=True)[:, :keep], True)
    choice = choice.masked_fill(~kept.repeat_interleave(per, dim=1), float("-inf"))
    idx = torch.argsort(choice, dim=-1, descending=True, stable=True)[:, :top]
    return idx, s.gather(1, idx)


def moe_ff(h, P, c):
    r = c["router"]
    n_real = int(r["experts"])
    idx, w = route(h, P, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(idx[t].tolist(), w[t]):
            out[t] += wt * (h[t] if e >= n_real else gated_expert(h[t:t + 1], P, "e%d." % e)[0])
    if c.get("shared"):
        out = out + gated_expert(h, P, "shared.")
    return out


def sub(tensors, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens):
    """-> (logits [T, vocab], [the residual stream after every layer])."""
    eps = float(cfg["norm"]["eps"])
    x = tensors["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    after = []
    for i, layer in enumerate(cfg["layers"]):
        pre = "l%d." % i
        assert layer["type"] == "parallel"
        m = layer["mixer"]
        y = float(m["left_scale"]) * left_attention(x, sub(tensors, pre + "mix.left."), m["left"], eps) \
            + float(m["right_scale"]) * right_memory(x, sub(tensors, pre + "mix.right."), m["right"], eps)
        x = x + rms(y, eps, tensors[pre + "norm1"].to(F64))
        mlp = layer.get("mlp")
        if mlp is not None:
            P = sub(tensors, pre + "mlp.")
            y = dense_ff(x, P) if mlp.get("kind", "dense") == "dense" else moe_ff(x, P, mlp)
            x = x + rms(y, eps, tensors[pre + "norm2"].to(F64))
        after.append(x)
    xn = rms(x, eps, tensors["final.norm"].to(F64))
    return xn @ tensors["embed"].to(F64).T, after

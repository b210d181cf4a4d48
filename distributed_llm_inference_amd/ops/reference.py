"""Plain PyTorch fp32 references of every HIP op (used by the numerics tests and by the CPU
stage executor). Shapes follow the kernels: activations are [tokens, features]."""
from __future__ import annotations

import math
import torch
import torch.nn.functional as F


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, unit_offset: bool = False) -> torch.Tensor:
    """`unit_offset`: the weight is stored as its distance from one (the scale is 1 + w)."""
    xf = x.float()
    return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * (w.float() + 1.0 if unit_offset else w.float())


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    return F.layer_norm(x.float(), (x.shape[-1],), w.float(), b.float(), eps)


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x.pow(3))))


def gemm(x, w, bias=None, residual=None, epi: int = 0):
    """epi as in the kernels: 0 none, 1 +bias, 2 +residual, 3 +bias+residual,
    4 swiglu (w = [gate; up] stacked, NOT interleaved), 5 +bias -> gelu_tanh."""
    y = x.float() @ w.float().t()
    if epi in (1, 3, 5):
        y = y + bias.float()
    if epi == 4:
        g, u = y.chunk(2, dim=-1)
        y = F.silu(g) * u
    if epi == 5:
        y = gelu_tanh(y)
    if epi in (2, 3):
        y = y + residual.float()
    return y


def rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """x [T, heads, D], half-split convention; cos/sin [P, D/2]."""
    d2 = x.shape[-1] // 2
    c = cos[positions.long()].unsqueeze(1).float()
    s = sin[positions.long()].unsqueeze(1).float()
    xf = x.float()
    a, b = xf[..., :d2], xf[..., d2:]
    return torch.cat([a * c - b * s, b * c + a * s], dim=-1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_pos0: int, scale: float,
              window: int = 0, sink: bool = False, k_pos0: int = 0, temp=None, dist_bias=None, sink_logit=None,
              keep_first: int = 0, softcap: float = 0.0, chunk: int = 0, head_mix=None) -> torch.Tensor:
    """One sequence. q [Tq, Hq, D] are the tokens at absolute positions q_pos0.., k [Tk, Hkv, D] and
    v [Tk, Hkv, Dv] hold positions k_pos0..k_pos0+Tk-1 (reaching at least the last query). Causal, GQA.
    `window` > 0: a query at i sees the keys j with 0 <= i - j < window. `sink`: the softmax's
    denominator has one more term, exp(0), that carries no value (`sink_logit` [Hq]: exp(sink_logit) instead).
    `temp` [Hq] multiplies a head's scaled scores; `dist_bias` [distances, Hq] is added to the scaled score of a
    key at distance i - j (after `temp`). `keep_first`: with a window, the keys at positions below it stay visible.
    `softcap` > 0: scaled scores become cap tanh(score / cap). `head_mix` [Hq, Hq]: the heads' scores (scaled, after
    `temp`) are mixed, s_h <- sum_g head_mix[h, g] s_g, before the mask. `chunk` > 0: a query sees only the keys of its own
    chunk of that many positions (counted from position 0). Returns [Tq, Hq, Dv] fp32."""
    Tq, Hq, D = q.shape
    Tk, Hkv, _ = k.shape
    g = Hq // Hkv
    kf = k.float().repeat_interleave(g, dim=1)
    vf = v.float().repeat_interleave(g, dim=1)
    s = torch.einsum("qhd,khd->hqk", q.float(), kf) * scale
    qpos = torch.arange(Tq, device=q.device).view(-1, 1) + q_pos0
    kpos = torch.arange(Tk, device=q.device).view(1, -1) + k_pos0
    if softcap > 0:
        s = softcap * torch.tanh(s / softcap)
    if temp is not None:
        s = s * temp.float().view(Hq, 1, 1)
    if dist_bias is not None:
        s = s + dist_bias.float()[(qpos - kpos).clamp(min=0)].permute(2, 0, 1)
    if head_mix is not None:
        s = torch.einsum("hg,gqk->hqk", head_mix.float(), s)
    hidden = kpos > qpos
    if chunk and chunk > 0:
        hidden = hidden | (torch.div(qpos, chunk, rounding_mode="floor") != torch.div(kpos, chunk, rounding_mode="floor"))
    if window and window > 0:
        hidden = hidden | ((qpos - kpos >= window) & (kpos >= keep_first))
    s = s.masked_fill(hidden.unsqueeze(0), float("-inf"))
    if sink:
        last = s.new_zeros(Hq, Tq, 1) if sink_logit is None else sink_logit.float().view(Hq, 1, 1).expand(Hq, Tq, 1)
        s = torch.cat([s, last], dim=-1)
        p = torch.softmax(s, dim=-1)[..., :-1]
    else:
        p = torch.softmax(s, dim=-1)
    return torch.einsum("hqk,khd->qhd", p, vf)


def short_conv(x: torch.Tensor, prev: torch.Tensor, taps: torch.Tensor):
    """Causal per-channel convolution over time. x [T, C] new inputs, prev [K-1, C] the inputs before them
    (zeros at a sequence's start), taps [C, K] with the last column on the current token. Returns
    (y [T, C] fp32, the last K-1 inputs)."""
    K = taps.shape[1]
    full = torch.cat([prev.float(), x.float()], dim=0)
    T = x.shape[0]
    y = sum(full[j:j + T] * taps[:, j].float() for j in range(K))
    return y, full[full.shape[0] - (K - 1):]


def l2_unit(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    xf = x.float()
    return xf * torch.rsqrt(xf.pow(2).sum(-1, keepdim=True) + eps)


def gated_delta_rule(q, k, v, beta, decay, S):
    """Token-by-token gated delta rule. q, k [T, G, d], v [T, H, dv], beta, decay [T, H], S [H, d, dv] fp32
    (head h reads q / k head h // (H / G)). Per token: S <- decay S; u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q. Returns (o [T, H, dv], S)."""
    T, H, _ = v.shape
    g = H // q.shape[1]
    qf, kf = q.float().repeat_interleave(g, dim=1), k.float().repeat_interleave(g, dim=1)
    vf, S = v.float(), S.float().clone()
    out = torch.empty(T, H, v.shape[2], dtype=torch.float32, device=v.device)
    for t in range(T):
        S = S * decay[t].float().view(H, 1, 1)
        u = beta[t].float().view(H, 1) * (vf[t] - torch.einsum("hdv,hd->hv", S, kf[t]))
        S = S + kf[t].unsqueeze(2) * u.unsqueeze(1)
        out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
    return out, S


def dyt(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, alpha) -> torch.Tensor:
    """Dynamic tanh in the place of a norm: tanh(alpha x) w + b, no statistics."""
    return torch.tanh(x.float() * float(alpha)) * w.float() + b.float()


def gelu_erf(x: torch.Tensor) -> torch.Tensor:
    return 0.5 * x * (1.0 + torch.erf(x * (2.0 ** -0.5)))


def distance_bias_table(rel: torch.Tensor, far: int, distances: int) -> torch.Tensor:
    """rel [rows, heads] (a learned bias per distance bucket and head) -> [distances, heads], the bias of every
    distance 0 .. distances-1 (`spec.distance_bucket` maps a distance to its row)."""
    from ..models.spec import distance_bucket
    rows = torch.tensor([distance_bucket(n, rel.shape[0], far) for n in range(distances)], dtype=torch.long, device=rel.device)
    return rel.float()[rows]


def general_delta_rule(r, k, v, w, a, S, eps: float = 1e-6):
    """Token by token, per head: u = k / sqrt(sum k^2 + eps); S <- diag(w) S - (a u) (u^T S) + k v^T (decay and removal
    both act on S as it was before the token); o = S^T r. r, k, v, w, a [T, H, d], S [H, d, d] fp32. Returns (o [T, H, d], S)."""
    rf, kf, vf, wf, af, S = r.float(), k.float(), v.float(), w.float(), a.float(), S.float().clone()
    u = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + eps)
    out = torch.empty_like(vf)
    for t in range(rf.shape[0]):
        us = torch.einsum("hd,hdv->hv", u[t], S)
        S = wf[t].unsqueeze(2) * S - (af[t] * u[t]).unsqueeze(2) * us.unsqueeze(1) + kf[t].unsqueeze(2) * vf[t].unsqueeze(1)
        out[t] = torch.einsum("hdv,hd->hv", S, rf[t])
    return out, S


def matrix_memory(q, k, v, log_i, log_f, S, n, m):
    """Token by token, per head: m' = max(log_f + m, log_i); S <- exp(log_f + m - m') S + exp(log_i - m') k v^T; n the
    same with k alone; o = S^T q / (max(|n . q|, exp(-m')) + 1e-6). q, k [T, H, d], v [T, H, dv], log_i, log_f [T, H],
    S [H, d, dv], n [H, d], m [H] fp32. Returns (o [T, H, dv], S, n, m)."""
    qf, kf, vf = q.float(), k.float(), v.float()
    S, n, m = S.float().clone(), n.float().clone(), m.float().clone()
    out = torch.empty_like(vf)
    for t in range(qf.shape[0]):
        new = torch.maximum(log_f[t].float() + m, log_i[t].float())
        keep, put = torch.exp(log_f[t].float() + m - new), torch.exp(log_i[t].float() - new)
        S = keep.view(-1, 1, 1) * S + put.view(-1, 1, 1) * kf[t].unsqueeze(2) * vf[t].unsqueeze(1)
        n = keep.view(-1, 1) * n + put.view(-1, 1) * kf[t]
        m = new
        den = torch.maximum((n * qf[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = torch.einsum("hdv,hd->hv", S, qf[t]) / den.view(-1, 1)
    return out, S, n, m


def moe_route(scores: torch.Tensor, top: int, groups: int, keep: int, scale: float, correction=None, group_rank: int = 2,
              renorm: bool = True):
    """scores [T, E] fp32 (sigmoids or a softmax of the router's logits) -> (experts [T, top] int64, weights [T, top] fp32).
    The choice goes by score + `correction` [E] (the score itself without one). Experts are split into `groups` contiguous
    blocks of equal size; a block is ranked by its best `group_rank` choice scores added up; experts outside the `keep` best
    blocks are out of the running (whatever their choice score's sign); of the rest the `top` highest are taken, each
    weighted by its score: score / (sum of the taken scores + 1e-20) * scale, or score * scale with `renorm` off. Equal
    choice scores go to the lower index."""
    T, E = scores.shape
    per = E // groups
    sf = scores.float()
    ch = sf if correction is None else sf + correction.float()
    gs = ch.view(T, groups, per).topk(min(group_rank, per), dim=-1).values.sum(-1)
    order = torch.argsort(gs, dim=-1, descending=True, stable=True)[:, :keep]
    allowed = torch.zeros(T, groups, dtype=torch.bool, device=scores.device).scatter_(1, order, True)
    masked = ch.masked_fill(~allowed.repeat_interleave(per, dim=1), float("-inf"))
    idx = torch.argsort(masked, dim=-1, descending=True, stable=True)[:, :top]
    val = sf.gather(1, idx)
    if not renorm:
        return idx, val * scale
    return idx, val / (val.sum(-1, keepdim=True) + 1e-20) * scale


def xielu(z: torch.Tensor, p, q) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z / 2; z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2."""
    zf = z.float()
    ap, aq = F.softplus(torch.as_tensor(p).float()), 0.5 + F.softplus(torch.as_tensor(q).float())
    return torch.where(zf > 0, ap * zf * zf + 0.5 * zf, aq * (torch.expm1(zf.clamp(max=0.0)) - zf) + 0.5 * zf)


def token_shift(h: torch.Tensor, prev: torch.Tensor, mu: torch.Tensor):
    """h [T, W] consecutive tokens of one sequence, prev [W] the h of the token before them (zeros at the start).
    Returns (h + (previous h - h) * mu, the last token's h)."""
    hf = h.float()
    before = torch.cat([prev.float().unsqueeze(0), hf[:-1]])
    return hf + (before - hf) * mu.float(), hf[-1]


def rope_partial(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, interleaved: bool) -> torch.Tensor:
    """x [T, heads, D]: the first 2 * cos.shape[1] entries of every vector are rotated by the token's position, pairs
    (2i, 2i + 1) when `interleaved`, else (i, i + dims / 2); the rest pass. fp32."""
    half = cos.shape[1]
    xf = x.float()
    head, tail = xf[..., :2 * half], xf[..., 2 * half:]
    c, s = cos[positions.long()].unsqueeze(1).float(), sin[positions.long()].unsqueeze(1).float()
    if interleaved:
        u, v = head[..., 0::2], head[..., 1::2]
        out = torch.stack([u * c - v * s, v * c + u * s], dim=-1).reshape(head.shape)
    else:
        u, v = head[..., :half], head[..., half:]
        out = torch.cat([u * c - v * s, v * c + u * s], dim=-1)
    return torch.cat([out, tail], dim=-1)


def block_linear(x: torch.Tensor, w: torch.Tensor, b=None) -> torch.Tensor:
    """x [T, blocks * n_in] through one matrix per block: w [blocks, n_out, n_in] (+ b [blocks, n_out]) -> [T, blocks * n_out], fp32."""
    nb, no, ni = w.shape
    y = torch.einsum("tbi,boi->tbo", x.float().reshape(-1, nb, ni), w.float())
    if b is not None:
        y = y + b.float()
    return y.reshape(-1, nb * no)


def rglru_scan(u: torch.Tensor, r: torch.Tensor, i: torch.Tensor, lam: torch.Tensor, S: torch.Tensor, c: float = 8.0):
    """Per channel: a = exp(-c r softplus(lam)); S <- a S + sqrt(1 - a^2) i u. u, r, i [T, W], lam, S [W] fp32.
    Returns (the state after every token [T, W], the last state)."""
    a = torch.exp(-c * r.float() * F.softplus(lam.float()))
    x = torch.sqrt(1.0 - a * a) * i.float() * u.float()
    S = S.float().clone()
    out = torch.empty_like(x)
    for t in range(x.shape[0]):
        S = a[t] * S + x[t]
        out[t] = S
    return out, S

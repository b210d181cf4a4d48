"""Helpers of the Tezesun tests: configurations and random weights made here, written as checkpoints (config.json +
model.safetensors), run through the package's own loader, executor and trace replay, and compared with the plain model of
`tezesun_oracle`."""
from __future__ import annotations

from typing import Dict, List, Optional

import numpy as np
import torch

import tezesun_oracle as O
from letarax_util import random_tokens, rel_err, replay, save_model, session  # noqa: F401  (shared checkpoint / replay helpers)


def rglru_layer(width: int, blocks: int, conv: int, ff: int = 64) -> dict:
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def attention_layer(heads: int, kv_heads: int, dim: int, vdim: int, window: Optional[int] = None, keep_first: int = 0,
                    scale: Optional[float] = None, softcap: float = 0.0, diff: float = 0.5, rot_dims: int = 0, base: float = 10000.0,
                    scaling: Optional[dict] = None, ff: int = 64) -> dict:
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5, "diff": diff}
    if softcap:
        m["softcap"] = softcap
    if window:
        m["mask"] = {"size": window, "keep_first": keep_first}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
        if scaling:
            m["rot"]["scaling"] = scaling
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def latent_layer(heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int, kv_rank: int, scale: Optional[float] = None,
                 base: float = 10000.0, ff: int = 64) -> dict:
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "rot": {"dims": rot_dim, "base": base}}
    return {"type": "latent_attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(layers: List[dict], vocab: int, width: int, eps: float = 1e-5, logit_scale: float = 1.0) -> dict:
    return {"architecture": "Tezesun", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width, "logit_scale": logit_scale}


def random_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bf16 tensors under the checkpoint's names, scaled so that every mechanism matters: projections at about
    1 / sqrt(fan-in), biases, gates, blends and layer scales of order one, decay rates spread over their range."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *shape, std=1.0: torch.randn(*shape, generator=g) * std
    W, H = {}, cfg["width"]
    W["embed"], W["head"], W["final.norm"] = rn(cfg["vocab"], H), rn(cfg["vocab"], H, std=2.0 * H ** -0.5), 1.0 + rn(H, std=0.1)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        W[p + "norm1"], W[p + "ls1"], W[p + "shift"] = 1.0 + rn(H, std=0.1), 0.5 + rn(H, std=0.15), torch.rand(H, generator=g)
        x = p + "mix."
        if l["type"] == "rglru":
            w, nb = m["width"], m["blocks"]
            bw = w // nb
            W[x + "y"], W[x + "y.b"], W[x + "x"], W[x + "x.b"] = rn(w, H, std=H ** -0.5), rn(w, std=0.3), rn(w, H, std=H ** -0.5), rn(w, std=0.3)
            W[x + "conv"], W[x + "conv.b"] = rn(w, m["conv"], std=0.6), rn(w, std=0.2)
            for gname in ("ra", "ri"):
                W[x + gname], W[x + gname + ".b"] = rn(nb, bw, bw, std=bw ** -0.5), rn(nb, bw, std=0.5)
            W[x + "lam"], n_o = rn(w, std=1.5) - 2.0, w
        elif l["type"] == "attention":
            hq, hk, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[x + "q"], W[x + "k"] = rn(hq * 2 * d, H, std=1.5 * H ** -0.5), rn(hk * 2 * d, H, std=1.5 * H ** -0.5)
            W[x + "v"], W[x + "g"] = rn(hk * dv, H, std=H ** -0.5), rn(hq * dv, H, std=H ** -0.5)
            for k in ("lq1", "lk1", "lq2", "lk2"):
                W[x + k] = rn(d, std=0.3)
            n_o = hq * dv
        else:
            hq, d, dr, dv, qr, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            W[x + "dq"], W[x + "dq.norm"], W[x + "uq"] = rn(qr, H, std=H ** -0.5), 1.0 + rn(qr, std=0.1), rn(hq * (d + dr), qr, std=1.5 * qr ** -0.5)
            W[x + "dkv"], W[x + "dkv.norm"] = rn(kr + dr, H, std=H ** -0.5), 1.0 + rn(kr, std=0.1)
            W[x + "uk"], W[x + "uv"] = rn(hq * d, kr, std=1.5 * kr ** -0.5), rn(hq * dv, kr, std=kr ** -0.5)
            n_o = hq * dv
        W[x + "o"] = rn(H, n_o, std=n_o ** -0.5)
        if l.get("mlp") is not None:
            ff = l["mlp"]["ff"]
            W[p + "ls2"] = 0.5 + rn(H, std=0.15)
            W[p + "mlp.up"], W[p + "mlp.down"], W[p + "mlp.act"] = rn(ff, H, std=H ** -0.5), rn(H, ff, std=ff ** -0.5), rn(2, std=0.5)
    return {k: v.to(torch.bfloat16) for k, v in W.items()}


def oracle_logits(cfg: dict, W, tokens: List[int]) -> np.ndarray:
    return O.forward(cfg, W, tokens)[0].numpy()


# Against the plain model: fp32 executors agree to rounding. In bf16 a tiny random model's worst position carries several
# per cent of rounding noise, so the sharp check of a bf16 run is `SAME`: however a request was cut into steps and whatever
# shared its batches, its logits agree with the same executor's run of the whole prompt alone to a few roundings.
TOL = {"fp32": 3e-4, "bf16": 0.3}
SAME = {"fp32": 1e-4, "bf16": 8e-2}


def alone(model_dir: str, backend: str, dtype: str, tokens: List[int]) -> np.ndarray:
    sess = session(model_dir, backend, dtype, max_tokens=len(tokens) + 64, slots=1)
    out = replay(sess, {"x": tokens}, [[("x", len(tokens))]])["x"]
    sess.close()
    return out


YARN = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}
R, A, L = rglru_layer, attention_layer, latent_layer
# Stacks that differ in everything a config can say: order and kinds of the layers, widths of the recurrent unit (equal to the
# model's or not), block counts (one block, blocks of one channel), tap counts from 1 up, head counts and groupings, key / value /
# latent sizes (equal, unequal, not powers of two), windows shorter and longer than a cache block or the prompts, kept first
# tokens (none, some, more than the window), rotated entries (all, some, none), rescaled or plain frequencies, soft caps or
# none, layers without a feed-forward, widths that are no multiple of 8, logit scales.
STACKS = {
    "mixed": make_config([L(4, 16, 8, 24, 32, 24), R(48, 4, 3), A(4, 2, 16, 32, window=20, keep_first=3, softcap=15.0, rot_dims=8, scaling=YARN),
                          R(48, 2, 4), L(2, 8, 8, 8, 16, 12, base=500.0)], vocab=96, width=48, logit_scale=1.7),
    "attn_first": make_config([A(2, 1, 8, 12, window=5, keep_first=9, rot_dims=8, base=200.0, ff=40), R(72, 1, 1, ff=0),
                               A(6, 3, 12, 8, window=37, keep_first=0, softcap=8.0, diff=0.2, rot_dims=4, scaling=YARN),
                               R(36, 36, 5), A(3, 3, 10, 20, scale=0.2, diff=0.7, ff=24)], vocab=70, width=36, eps=1e-6),
    "only_rglru": make_config([R(64, 4, 4), R(128, 8, 2, ff=32), R(32, 2, 3, ff=0)], vocab=64, width=64),
    "only_latent": make_config([L(3, 12, 4, 20, 24, 18, scale=0.4), L(1, 32, 16, 8, 40, 48, ff=0), L(4, 8, 2, 8, 8, 8)], vocab=51, width=40, logit_scale=0.5),
    # widths and inner sizes that the packed-weight GEMMs take in bf16 (multiples of 128)
    "packed": make_config([L(4, 32, 16, 32, 128, 48), R(128, 2, 4, ff=128), A(4, 2, 32, 64, window=44, keep_first=4, softcap=25.0, rot_dims=16,
                                                                              scaling=YARN, ff=256), R(256, 4, 3, ff=128)], vocab=90, width=128, logit_scale=2.5),
}

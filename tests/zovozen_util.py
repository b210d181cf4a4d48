"""Helpers of the Zovozen tests: configurations and random weights made here, written as checkpoints (config.json +
model.safetensors), run through the package's own loader, executor and trace replay, and compared with the plain model of
`zovozen_oracle`."""
from __future__ import annotations

from typing import Dict, List, Optional

import numpy as np
import torch

import zovozen_oracle as O
from letarax_util import random_tokens, rel_err, replay, save_model, session  # noqa: F401  (shared checkpoint / replay helpers)


def dense(ff: int) -> dict:
    return {"kind": "dense", "ff": ff}


def moe(experts: int, top: int, ff: int, identity: int = 0, groups: int = 1, keep: Optional[int] = None, shared: int = 0) -> dict:
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "identity": identity,
                                                         "groups": {"count": groups, "keep": keep if keep is not None else groups}}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(heads: int, kv_heads: int, dim: int, vdim: int, mem: tuple, chunk: int = 0, rot_dims: int = 0, base: float = 10000.0,
          factor: float = 1.0, scale: Optional[float] = None, scales: tuple = (0.7, 0.6), cap: float = 12.0, mlp: Optional[dict] = None) -> dict:
    """`mem`: (heads, dim, vdim) of the matrix memory beside the attention."""
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if chunk:
        left["mask"] = {"size": chunk}
    if rot_dims:
        left["rot"] = {"dims": rot_dims, "base": base}
        if factor != 1.0:
            left["rot"]["scaling"] = {"factor": factor}
    right = {"heads": mem[0], "dim": mem[1], "vdim": mem[2], "gate_cap": cap}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": scales[0], "right_scale": scales[1]}, "mlp": mlp}


def make_config(layers: List[dict], vocab: int, width: int, eps: float = 1e-5) -> dict:
    return {"architecture": "Zovozen", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bf16 tensors under the checkpoint's names, scaled so that every mechanism matters: projections at about 1 / sqrt(fan-in),
    biases, norm weights, temperatures, head mixes, sinks, gate biases and routing corrections of order one (of the order of a
    score for the corrections)."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *shape, std=1.0: torch.randn(*shape, generator=g) * std
    W, H = {}, cfg["width"]
    W["embed"], W["final.norm"] = rn(cfg["vocab"], H), 1.0 + rn(H, std=0.1)
    for i, l in enumerate(cfg["layers"]):
        p, a, b = f"l{i}.", l["mixer"]["left"], l["mixer"]["right"]
        W[p + "norm1"] = 1.0 + rn(H, std=0.2)
        x = p + "mix.left."
        hq, hk, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        for n, rows in (("q", hq * d), ("k", hk * d), ("v", hk * dv)):
            W[x + n], W[x + n + ".b"] = rn(rows, H, std=1.5 * H ** -0.5), rn(rows, std=0.3)
        W[x + "q.norm"], W[x + "k.norm"] = 1.0 + rn(hq * d, std=0.2), 1.0 + rn(hk * d, std=0.2)
        W[x + "talk"], W[x + "temp"], W[x + "sink"] = torch.eye(hq) + rn(hq, hq, std=0.3), 1.0 + rn(hq, std=0.3), rn(hq)
        W[x + "g"], W[x + "o"], W[x + "o.b"] = rn(hq * dv, H, std=H ** -0.5), rn(H, hq * dv, std=(hq * dv) ** -0.5), rn(H, std=0.2)
        x = p + "mix.right."
        bh, bd, bv = b["heads"], b["dim"], b["vdim"]
        W[x + "q"], W[x + "k"], W[x + "v"] = rn(bh * bd, H, std=H ** -0.5), rn(bh * bd, H, std=H ** -0.5), rn(bh * bv, H, std=H ** -0.5)
        W[x + "g"], W[x + "o"], W[x + "norm"] = rn(bh * bv, H, std=H ** -0.5), rn(H, bh * bv, std=(bh * bv) ** -0.5), 1.0 + rn(bh * bv, std=0.1)
        for n in ("i", "f"):
            W[x + n], W[x + n + ".b"] = rn(bh, H, std=2.0 * H ** -0.5), rn(bh) + (2.0 if n == "f" else 0.0)
        mlp = l.get("mlp")
        if mlp is None:
            continue
        W[p + "norm2"] = 1.0 + rn(H, std=0.2)
        x = p + "mlp."
        if mlp["kind"] == "dense":
            ff = mlp["ff"]
            W[x + "up"], W[x + "up.b"], W[x + "down"], W[x + "down.b"] = rn(ff, H, std=H ** -0.5), rn(ff, std=0.3), rn(H, ff, std=ff ** -0.5), rn(H, std=0.2)
        else:
            r, ff = mlp["router"], mlp["expert"]["ff"]
            outs = r["experts"] + r.get("identity", 0)
            W[x + "router"], W[x + "correction"] = rn(outs, H, std=2.0 * H ** -0.5), rn(outs, std=0.5 / outs)
            for e in [f"e{j}." for j in range(r["experts"])] + (["shared."] if mlp.get("shared") else []):
                f = mlp["shared"]["ff"] if e == "shared." else ff
                W[x + e + "gate"], W[x + e + "up"], W[x + e + "down"] = rn(f, H, std=1.5 * H ** -0.5), rn(f, H, std=1.5 * H ** -0.5), rn(H, f, std=f ** -0.5)
    return {k: v.to(torch.bfloat16) for k, v in W.items()}


def oracle_logits(cfg: dict, W, tokens: List[int]) -> np.ndarray:
    return O.forward(cfg, W, tokens)[0].numpy()


# Against the plain model: fp32 executors agree to rounding. In bf16 a tiny random model's worst position carries several
# per cent of rounding noise (and a router is a discontinuity: where two experts nearly tie, one rounding moves a whole
# position), so the sharp check of a bf16 run is `SAME`: however a request was cut into steps and whatever shared its
# batches, its logits agree with the same executor's run of the whole prompt alone to a few roundings.
TOL = {"fp32": 3e-4, "bf16": 0.3}
SAME = {"fp32": 1e-4, "bf16": 8e-2}


def alone(model_dir: str, backend: str, dtype: str, tokens: List[int]) -> np.ndarray:
    sess = session(model_dir, backend, dtype, max_tokens=len(tokens) + 64, slots=1)
    out = replay(sess, {"x": tokens}, [[("x", len(tokens))]])["x"]
    sess.close()
    return out


Z = layer
# Stacks that differ in everything a config can say: head counts and groupings of the attention (one key / value head, as many
# as heads, groups of 2 and 3), head counts of the memory (equal to the attention's or not, a single head), key / value sizes
# (equal, unequal, not powers of two, no multiples of 8), chunks shorter and longer than a cache block or the prompts or absent,
# rotated entries (all, some, none) with plain or rescaled frequencies, branch weights, gate caps, the feed-forward of every
# layer (none, dense, routed with or without identity experts, groups and a shared expert; one chosen expert; groups of one),
# widths that are no multiple of 8, eps.
STACKS = {
    "mixed": make_config([Z(4, 2, 16, 24, (2, 8, 16), chunk=20, rot_dims=8, base=5000.0, factor=4.0, mlp=dense(40)),
                          Z(4, 2, 16, 24, (2, 8, 16), chunk=20, rot_dims=8, base=5000.0, factor=4.0, mlp=moe(6, 2, 24, identity=2, groups=4, keep=2, shared=32)),
                          Z(6, 3, 8, 8, (3, 16, 8), chunk=33, rot_dims=8, scale=0.5, scales=(1.2, 0.3), mlp=None),
                          Z(2, 1, 24, 12, (1, 12, 20), chunk=7, rot_dims=4, base=100.0, cap=6.0, mlp=moe(5, 1, 16, identity=0, groups=1, shared=0))],
                         vocab=96, width=48),
    "odd_sizes": make_config([Z(3, 3, 10, 6, (2, 7, 9), chunk=0, rot_dims=10, factor=2.0, scales=(0.5, 1.0), mlp=moe(4, 3, 12, identity=2, groups=3, keep=2, shared=20)),
                              Z(4, 1, 12, 20, (5, 4, 6), chunk=64, rot_dims=0, scale=0.3, mlp=dense(56)),
                              Z(1, 1, 36, 20, (4, 10, 10), chunk=1, rot_dims=2, mlp=moe(6, 2, 8, identity=0, groups=6, keep=3, shared=8))],
                             vocab=51, width=36, eps=1e-6),
    # widths and inner sizes that the packed-weight GEMMs and the matrix-core attention take in bf16
    "packed": make_config([Z(4, 2, 32, 64, (2, 32, 64), chunk=44, rot_dims=16, factor=6.0, mlp=moe(8, 2, 64, identity=2, groups=5, keep=2, shared=96)),
                           Z(8, 2, 16, 32, (4, 64, 32), chunk=100, rot_dims=16, base=500000.0, mlp=dense(256)),
                           Z(4, 4, 64, 40, (2, 32, 64), chunk=32, rot_dims=32, mlp=moe(4, 2, 128, identity=4, groups=2, keep=2, shared=0))],
                          vocab=90, width=128),
}

"""Per-stage weights in the engine's logical layout.

Logical layout (all matrices `[out_features, in_features]`, i.e. what ``nn.Linear`` stores):

  embed        [V, H]            stage 0 (and the last stage when lm_head is tied)
  pos_embed    [P, H]            GPT-2 only, stage 0
  layers[i]:   ln1_w (+ln1_b)    [H]
               w_qkv (+b_qkv)    [Hq*D + 2*Hkv*D, H]     q,k,v concatenated -> one GEMM
               w_o   (+b_o)      [H, Hq*D]
               ln2_w (+ln2_b)    [H]
               w_gate, w_up      [I, H]  (Llama)   |  w_fc (+b_fc) [I, H]  (GPT-2)
               w_down (+b_down)  [H, I]
  final_norm_w (+final_norm_b)   [H]     last stage
  lm_head      [V, H]            last stage (aliases `embed` data when tied)

Hybrid stacks (`spec.layer_specs`, the Letarax checkpoint names ``embed``, ``l{i}.norm1`` / ``norm1b`` /
``norm2`` / ``norm2b``, ``l{i}.mix.*``, ``l{i}.mlp.*``, ``final.norm``) use per layer:

               ln1_w, ln1b_w     [H]     norm before / after the mixer (stored as the distance from one)
  attention:   w_qkv, b_qkv      [Hq*d + G*d + G*dv, H]  q, k, v concatenated
               vmix              []      blend weight of the value mixing
  delta:       w_in              [G*d + G*d + Hv*dv + Hv*dv + Hv + Hv, H]   q, k, v, output gate, beta, decay
               conv_w            [G*d + G*d + Hv*dv, taps]                    causal convolutions of q, k, v
               A_log, dt_bias    [Hv]    o_norm_w [dv]
               w_o               [H, heads*dv]
  feed-forward ln2_w, ln2b_w, w_gate, b_gate, w_up, b_up [I, H] / [I], w_down, b_down
  lm_head = embed.

A stage materialises only what its `StagePlan` owns.  The reference instead loads the full
model in every process (orchestration.py:39-47, Worker1.py:60-75).

HF tensor names honoured — Llama: ``model.embed_tokens.weight``,
``model.layers.{i}.{input_layernorm,post_attention_layernorm}.weight``,
``model.layers.{i}.self_attn.{q,k,v,o}_proj.weight``,
``model.layers.{i}.mlp.{gate,up,down}_proj.weight``, ``model.norm.weight``, ``lm_head.weight``.
GPT-2 (optionally prefixed ``transformer.``): ``wte``, ``wpe``, ``h.{i}.ln_{1,2}``,
``h.{i}.attn.c_attn`` / ``c_proj``, ``h.{i}.mlp.c_fc`` / ``c_proj`` (Conv1D: stored
``[in, out]`` and therefore transposed here), ``ln_f``.
"""
from __future__ import annotations

import hashlib
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

from .partition import StagePlan
from .safetensors_io import CheckpointReader
from .spec import ModelSpec


@dataclass
class StageWeights:
    spec: ModelSpec
    plan: StagePlan
    embed: Optional[torch.Tensor] = None
    pos_embed: Optional[torch.Tensor] = None
    layers: List[Dict[str, torch.Tensor]] = field(default_factory=list)
    final_norm_w: Optional[torch.Tensor] = None
    final_norm_b: Optional[torch.Tensor] = None
    lm_head: Optional[torch.Tensor] = None
    final_norm_a: Optional[torch.Tensor] = None      # dynamic-tanh norms: the scalar inside the tanh
    loop_step: Optional[torch.Tensor] = None         # [passes, H]: added to the residual stream ahead of each pass of a repeated stretch

    def num_bytes(self) -> int:
        seen, total = set(), 0
        for t in self.tensors():
            p = t.untyped_storage().data_ptr()
            if p in seen:
                continue
            seen.add(p)
            total += t.numel() * t.element_size()
        return total

    def tensors(self):
        for t in (self.embed, self.pos_embed, self.final_norm_w, self.final_norm_b, self.lm_head, self.final_norm_a, self.loop_step):
            if t is not None:
                yield t
        for l in self.layers:
            yield from l.values()

    def to(self, device=None, dtype=None) -> "StageWeights":
        def cv(t):
            if t is None:
                return None
            return t.to(device=device, dtype=dtype if t.is_floating_point() else None)
        tied = self.lm_head is not None and self.embed is not None and \
            self.lm_head.data_ptr() == self.embed.data_ptr()
        out = StageWeights(self.spec, self.plan)
        out.embed = cv(self.embed)
        out.pos_embed = cv(self.pos_embed)
        out.layers = [{k: cv(v) for k, v in l.items()} for l in self.layers]
        out.final_norm_w = cv(self.final_norm_w)
        out.final_norm_b = cv(self.final_norm_b)
        out.final_norm_a, out.loop_step = cv(self.final_norm_a), cv(self.loop_step)
        out.lm_head = out.embed if tied else cv(self.lm_head)
        return out


# --------------------------------------------------------------------------------------
# random initialisation (benchmarks and tests: no checkpoint, no network)
# --------------------------------------------------------------------------------------

def _seed_for(name: str, seed: int) -> int:
    h = hashlib.blake2b(f"{seed}:{name}".encode(), digest_size=8).digest()
    return int.from_bytes(h, "little") & 0x7FFF_FFFF_FFFF_FFFF


def _randn(name, shape, seed, device, dtype, std=0.02):
    """Deterministic per-tensor init: the value of a tensor depends only on (seed, name),
    never on which stage materialises it, so any partition of the model sees the same weights."""
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(_seed_for(name, seed))
    gen_dtype = torch.float32 if dev.type == "cpu" else dtype
    t = torch.empty(shape, device=dev, dtype=gen_dtype)
    t.normal_(0.0, std, generator=g)
    return t.to(dtype)


# ---- Nufapel: checkpoint names <-> the logical layout --------------------------------------------------------------
# Per layer: ln1_w / ln1_b / ln1_a (and ln2_*) dynamic-tanh norms; w_rg1 / b_rg1 (w_rg2 / b_rg2) residual gates;
#   general_delta: w_in = r | k | v | g | a | w1 (one GEMM), b_a, w_w2 [heads dim, rank], w0, o_norm_w, w_o
#   parallel:      w_in = left q | k | v | g, right q | k | v | g | i | f; rel [rows, heads], temp, sink, w_o (left);
#                  b_if, o_norm_w, w_o_r (right); out_l, out_r (the branches' RMS weights)
#   dense:         w_up, w_down            moe: w_router [E, H], w_gate_e / w_up_e [E, ff, H], w_down_e [E, H, ff]
_GD_IN = ("r", "k", "v", "g", "a", "w1")
_PAR_IN = ("left.q", "left.k", "left.v", "left.g", "right.q", "right.k", "right.v", "right.g", "right.i", "right.f")


def _nufapel_layer_names(ls, p: str) -> Dict[str, object]:
    """logical name -> checkpoint name, or a tuple of names that are concatenated (dim 0) or stacked (experts)."""
    m, f = p + "mix.", p + "mlp."
    n: Dict[str, object] = {"ln1_w": p + "norm1", "ln1_b": p + "norm1.b", "ln1_a": p + "norm1.alpha", "w_rg1": p + "rg1", "b_rg1": p + "rg1.b"}
    if ls.kind == "general_delta":
        n.update({"w_in": tuple(m + x for x in _GD_IN), "b_a": m + "a.b", "w_w2": m + "w2", "w0": m + "w0", "o_norm_w": m + "norm", "w_o": m + "o"})
    else:
        n.update({"w_in": tuple(m + x for x in _PAR_IN), "rel": m + "left.rel", "temp": m + "left.temp", "sink": m + "left.sink",
                  "w_o": m + "left.o", "b_if": (m + "right.i.b", m + "right.f.b"), "o_norm_w": m + "right.norm", "w_o_r": m + "right.o",
                  "out_l": m + "left.out", "out_r": m + "right.out"})
    if ls.has_ff:
        n.update({"ln2_w": p + "norm2", "ln2_b": p + "norm2.b", "ln2_a": p + "norm2.alpha", "w_rg2": p + "rg2", "b_rg2": p + "rg2.b"})
        if ls.moe is not None:
            n["w_router"] = f + "router"
            for x in ("gate", "up", "down"):
                n[f"w_{x}_e"] = [f"{f}e{e}.{x}" for e in range(ls.moe.experts)]
        else:
            n.update({"w_up": f + "up", "w_down": f + "down"})
    return n


def _load_nufapel_weights(rd, spec: ModelSpec, plan: StagePlan, device, dtype) -> StageWeights:
    w = StageWeights(spec, plan)
    get = lambda name: rd.get(name).to(device=device, dtype=dtype)
    w.embed, w.pos_embed, w.lm_head = get("embed"), get("pos"), get("head")
    w.final_norm_w, w.final_norm_b, w.final_norm_a = get("final.norm"), get("final.norm.b"), get("final.norm.alpha").reshape(())
    if spec.loop:
        w.loop_step = get("loop.step")
    for i in plan.layers:
        l = {}
        for k, names in _nufapel_layer_names(spec.layer_specs[i], f"l{i}.").items():
            if isinstance(names, tuple):
                l[k] = torch.cat([get(x) for x in names], dim=0)
            elif isinstance(names, list):
                l[k] = torch.stack([get(x) for x in names], dim=0)
            else:
                l[k] = get(names)
        w.layers.append(l)
    return w


def _nufapel_in_sizes(ls, l) -> List[int]:
    if ls.kind == "general_delta":
        n = ls.heads * ls.dim
        return [n] * 5 + [l["w_w2"].shape[1]]
    a, b = ls.branches
    return [a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim, a.heads, b.heads * b.dim, b.heads * b.dim, b.heads * b.vdim,
            b.heads * b.vdim, b.heads, b.heads]


def export_nufapel_state_dict(w: StageWeights) -> Dict[str, torch.Tensor]:
    """Logical -> checkpoint names (tests, `save` of random models)."""
    spec = w.spec
    sd = {"embed": w.embed, "pos": w.pos_embed, "head": w.lm_head, "final.norm": w.final_norm_w, "final.norm.b": w.final_norm_b,
          "final.norm.alpha": w.final_norm_a}
    if w.loop_step is not None:
        sd["loop.step"] = w.loop_step
    for i, l in zip(w.plan.layers, w.layers):
        ls = spec.layer_specs[i]
        for k, names in _nufapel_layer_names(ls, f"l{i}.").items():
            if isinstance(names, tuple):
                sizes = _nufapel_in_sizes(ls, l) if k == "w_in" else [l[k].shape[0] // len(names)] * len(names)
                for x, t in zip(names, torch.split(l[k], sizes)):
                    sd[x] = t
            elif isinstance(names, list):
                for x, t in zip(names, l[k]):
                    sd[x] = t
            else:
                sd[names] = l[k]
    return {k: v.detach().clone().contiguous() for k, v in sd.items()}


def _random_nufapel_weights(spec: ModelSpec, plan: StagePlan, seed: int, device, dtype) -> StageWeights:
    """Random weights with which every mechanism matters: projections at 1 / sqrt(fan-in), gates, biases, sinks,
    temperatures and distance biases of order one, decays spread over their range."""
    H, V = spec.hidden_size, spec.vocab_size
    w = StageWeights(spec, plan)
    rn = lambda name, shape, std: _randn(name, shape, seed, device, dtype, std=std)
    one = lambda name, shape, std: torch.ones(shape, device=device, dtype=dtype) + rn(name, shape, std)
    w.embed, w.pos_embed, w.lm_head = rn("embed", (V, H), 1.0), rn("pos", (spec.max_position, H), 0.5), rn("head", (V, H), 2.0 * H ** -0.5)
    w.final_norm_w, w.final_norm_b = one("final.norm", (H,), 0.1), rn("final.norm.b", (H,), 0.1)
    w.final_norm_a = torch.tensor(0.6, device=device, dtype=dtype)
    if spec.loop:
        w.loop_step = rn("loop.step", (spec.loop[2], H), 0.5)
    for i in plan.layers:
        ls, p = spec.layer_specs[i], f"layers.{i}."
        l: Dict[str, torch.Tensor] = {}
        for s_ in ("1", "2") if ls.has_ff else ("1",):
            l[f"ln{s_}_w"], l[f"ln{s_}_b"] = one(p + f"ln{s_}_w", (H,), 0.1), rn(p + f"ln{s_}_b", (H,), 0.1)
            l[f"ln{s_}_a"] = torch.tensor(0.4 + 0.05 * ((i + int(s_)) % 5), device=device, dtype=dtype)
            l[f"w_rg{s_}"], l[f"b_rg{s_}"] = rn(p + f"w_rg{s_}", (H, H), H ** -0.5), rn(p + f"b_rg{s_}", (H,), 0.5)
        if ls.kind == "general_delta":
            n, R = ls.heads * ls.dim, ls.rank or 16
            l["w_in"] = torch.cat([rn(p + "w_in", (5 * n, H), H ** -0.5), rn(p + "w_w1", (R, H), H ** -0.5)])
            l["b_a"], l["w_w2"], l["w0"] = rn(p + "b_a", (n,), 0.5), rn(p + "w_w2", (n, R), 2.0 * R ** -0.5), rn(p + "w0", (n,), 1.5)
            l["o_norm_w"], l["w_o"] = one(p + "o_norm_w", (n,), 0.1), rn(p + "w_o", (H, n), n ** -0.5)
        else:
            a, b = ls.branches
            rows = a.bias_rows or 16
            sizes = _nufapel_in_sizes(ls, None)
            l["w_in"] = rn(p + "w_in", (sum(sizes), H), H ** -0.5)
            l["rel"], l["temp"], l["sink"] = rn(p + "rel", (rows, a.heads), 1.0), one(p + "temp", (a.heads,), 0.3), rn(p + "sink", (a.heads,), 1.0)
            l["w_o"] = rn(p + "w_o", (H, a.heads * a.vdim), (a.heads * a.vdim) ** -0.5)
            l["b_if"] = rn(p + "b_if", (2 * b.heads,), 1.0)
            l["o_norm_w"], l["w_o_r"] = one(p + "o_norm_w", (b.heads * b.vdim,), 0.1), rn(p + "w_o_r", (H, b.heads * b.vdim), (b.heads * b.vdim) ** -0.5)
            l["out_l"], l["out_r"] = one(p + "out_l", (H,), 0.1), one(p + "out_r", (H,), 0.1)
        if ls.moe is not None:
            e = ls.moe
            l["w_router"] = rn(p + "w_router", (e.experts, H), 2.0 * H ** -0.5)
            l["w_gate_e"], l["w_up_e"] = rn(p + "w_gate_e", (e.experts, e.ff, H), 1.5 * H ** -0.5), rn(p + "w_up_e", (e.experts, e.ff, H), 1.5 * H ** -0.5)
            l["w_down_e"] = rn(p + "w_down_e", (e.experts, H, e.ff), e.ff ** -0.5)
        elif ls.ff:
            l["w_up"], l["w_down"] = rn(p + "w_up", (ls.ff, H), H ** -0.5), rn(p + "w_down", (H, ls.ff), ls.ff ** -0.5)
        w.layers.append(l)
    return w


# ---- Tezesun: checkpoint names <-> the logical layout ----------------------------------------------------------------
# Per layer: ln1_w (the one norm), ls1 / ls2 (layer scales of mixer / feed-forward), shift (token-shift blend);
#   rglru:            w_in = y | x (one GEMM) with b_in, conv_w [W, taps], conv_b, w_ra / w_ri [blocks, bw, bw] with b_ra / b_ri, lam, w_o
#   attention:        w_in = q | k | v | g (one GEMM), lq1, lk1, lq2, lk2, w_o
#   latent_attention: w_in = dq | dkv (one GEMM), dq_norm, dkv_norm, w_uq, w_uk, w_uv, w_o
#   feed-forward:     w_up, w_down, act (the two numbers of the activation)
def _tezesun_layer_names(ls, p: str) -> Dict[str, object]:
    m, f = p + "mix.", p + "mlp."
    n: Dict[str, object] = {"ln1_w": p + "norm1", "ls1": p + "ls1", "shift": p + "shift", "w_o": m + "o"}
    if ls.kind == "rglru":
        n.update({"w_in": (m + "y", m + "x"), "b_in": (m + "y.b", m + "x.b"), "conv_w": m + "conv", "conv_b": m + "conv.b",
                  "w_ra": m + "ra", "b_ra": m + "ra.b", "w_ri": m + "ri", "b_ri": m + "ri.b", "lam": m + "lam"})
    elif ls.kind == "attention":
        n.update({"w_in": (m + "q", m + "k", m + "v", m + "g"), "lq1": m + "lq1", "lk1": m + "lk1", "lq2": m + "lq2", "lk2": m + "lk2"})
    else:
        n.update({"w_in": (m + "dq", m + "dkv"), "dq_norm": m + "dq.norm", "dkv_norm": m + "dkv.norm", "w_uq": m + "uq",
                  "w_uk": m + "uk", "w_uv": m + "uv"})
    if ls.ff:
        n.update({"ls2": p + "ls2", "w_up": f + "up", "w_down": f + "down", "act": f + "act"})
    return n


def _tezesun_in_sizes(ls) -> List[int]:
    if ls.kind == "rglru":
        return [ls.rec_width, ls.rec_width]
    if ls.kind == "attention":
        return [ls.heads * ls.maps * ls.dim, ls.kv_heads * ls.maps * ls.dim, ls.kv_heads * ls.vdim, ls.heads * ls.vdim]
    return [ls.q_rank, ls.kv_rank + ls.rot_dim]


def _load_tezesun_weights(rd, spec: ModelSpec, plan: StagePlan, device, dtype) -> StageWeights:
    w = StageWeights(spec, plan)
    get = lambda name: rd.get(name).to(device=device, dtype=dtype)
    w.embed, w.lm_head, w.final_norm_w = get("embed"), get("head"), get("final.norm")
    for i in plan.layers:
        l = {}
        for k, names in _tezesun_layer_names(spec.layer_specs[i], f"l{i}.").items():
            l[k] = torch.cat([get(x) for x in names], dim=0) if isinstance(names, tuple) else get(names)
        w.layers.append(l)
    return w


def export_tezesun_state_dict(w: StageWeights) -> Dict[str, torch.Tensor]:
    """Logical -> checkpoint names (tests, `save` of random models)."""
    spec = w.spec
    sd = {"embed": w.embed, "head": w.lm_head, "final.norm": w.final_norm_w}
    for i, l in zip(w.plan.layers, w.layers):
        ls = spec.layer_specs[i]
        for k, names in _tezesun_layer_names(ls, f"l{i}.").items():
            if isinstance(names, tuple):
                for x, t in zip(names, torch.split(l[k], _tezesun_in_sizes(ls))):
                    sd[x] = t
            else:
                sd[names] = l[k]
    return {k: v.detach().clone().contiguous() for k, v in sd.items()}


def _random_tezesun_weights(spec: ModelSpec, plan: StagePlan, seed: int, device, dtype) -> StageWeights:
    """Random weights with which every mechanism matters: projections at 1 / sqrt(fan-in), biases, gates, layer scales
    and blends of order one, decays spread over their range."""
    H, V = spec.hidden_size, spec.vocab_size
    w = StageWeights(spec, plan)
    rn = lambda name, shape, std: _randn(name, shape, seed, device, dtype, std=std)
    one = lambda name, shape, std: torch.ones(shape, device=device, dtype=dtype) + rn(name, shape, std)
    w.embed, w.lm_head, w.final_norm_w = rn("embed", (V, H), 1.0), rn("head", (V, H), H ** -0.5), one("final.norm", (H,), 0.1)
    for i in plan.layers:
        ls, p = spec.layer_specs[i], f"layers.{i}."
        l: Dict[str, torch.Tensor] = {"ln1_w": one(p + "ln1_w", (H,), 0.1), "ls1": one(p + "ls1", (H,), 0.3) * 0.5,
                                      "shift": (rn(p + "shift", (H,), 0.25) + 0.5).clamp(0.0, 1.0)}
        l["w_in"] = rn(p + "w_in", (sum(_tezesun_in_sizes(ls)), H), H ** -0.5)
        if ls.kind == "rglru":
            W, nb, bw = ls.rec_width, ls.blocks, ls.rec_width // ls.blocks
            l["b_in"], l["conv_w"], l["conv_b"] = rn(p + "b_in", (2 * W,), 0.2), rn(p + "conv_w", (W, ls.conv), 0.6), rn(p + "conv_b", (W,), 0.2)
            l["w_ra"], l["b_ra"] = rn(p + "w_ra", (nb, bw, bw), bw ** -0.5), rn(p + "b_ra", (nb, bw), 0.5)
            l["w_ri"], l["b_ri"] = rn(p + "w_ri", (nb, bw, bw), bw ** -0.5), rn(p + "b_ri", (nb, bw), 0.5)
            l["lam"], n_o = rn(p + "lam", (W,), 1.5) - 2.0, W
        elif ls.kind == "attention":
            for k in ("lq1", "lk1", "lq2", "lk2"):
                l[k] = rn(p + k, (ls.dim,), 0.3)
            n_o = ls.heads * ls.vdim
        else:
            l["dq_norm"], l["dkv_norm"] = one(p + "dq_norm", (ls.q_rank,), 0.1), one(p + "dkv_norm", (ls.kv_rank,), 0.1)
            l["w_uq"] = rn(p + "w_uq", (ls.heads * (ls.dim + ls.rot_dim), ls.q_rank), 2.0 * ls.q_rank ** -0.5)
            l["w_uk"] = rn(p + "w_uk", (ls.heads * ls.dim, ls.kv_rank), 2.0 * ls.kv_rank ** -0.5)
            l["w_uv"] = rn(p + "w_uv", (ls.heads * ls.vdim, ls.kv_rank), ls.kv_rank ** -0.5)
            n_o = ls.heads * ls.vdim
        l["w_o"] = rn(p + "w_o", (H, n_o), n_o ** -0.5)
        if ls.ff:
            l["ls2"] = one(p + "ls2", (H,), 0.3) * 0.5
            l["w_up"], l["w_down"] = rn(p + "w_up", (ls.ff, H), H ** -0.5), rn(p + "w_down", (H, ls.ff), ls.ff ** -0.5)
            l["act"] = rn(p + "act", (2,), 0.5)
        w.layers.append(l)
    return w

# ---- Zovozen: checkpoint names <-> the logical layout ----------------------------------------------------------------
# Per layer: ln1_w / ln2_w (the norms on the sublayers' outputs);
#   mixer:  w_in = left q | k | v | g, right q | k | v | g | i | f (one GEMM), b_qkv (left q | k | v), q_norm_w, k_norm_w,
#           talk [heads, heads], temp, sink, w_o / b_o (left); b_if, o_norm_w, w_o_r (right)
#   dense:  w_up / b_up, w_down / b_down
#   moe:    w_router [experts + identity, H], correction, w_gate_e / w_up_e [E, ff, H], w_down_e [E, H, ff],
#           shared expert w_gate_s / w_up_s / w_down_s
def _zovozen_layer_names(ls, p: str) -> Dict[str, object]:
    """logical name -> checkpoint name, or a tuple of names that are concatenated (dim 0), or a list that is stacked (experts)."""
    m, f = p + "mix.", p + "mlp."
    n: Dict[str, object] = {
        "ln1_w": p + "norm1", "w_in": tuple(m + x for x in _PAR_IN), "b_qkv": (m + "left.q.b", m + "left.k.b", m + "left.v.b"),
        "q_norm_w": m + "left.q.norm", "k_norm_w": m + "left.k.norm", "talk": m + "left.talk", "temp": m + "left.temp",
        "sink": m + "left.sink", "w_o": m + "left.o", "b_o": m + "left.o.b", "b_if": (m + "right.i.b", m + "right.f.b"),
        "o_norm_w": m + "right.norm", "w_o_r": m + "right.o"}
    if ls.has_ff:
        n["ln2_w"] = p + "norm2"
        if ls.moe is not None:
            n.update({"w_router": f + "router", "correction": f + "correction"})
            for x in ("gate", "up", "down"):
                n[f"w_{x}_e"] = [f"{f}e{e}.{x}" for e in range(ls.moe.experts)]
                if ls.moe.shared_ff:
                    n[f"w_{x}_s"] = f"{f}shared.{x}"
        else:
            n.update({"w_up": f + "up", "b_up": f + "up.b", "w_down": f + "down", "b_down": f + "down.b"})
    return n


def _zovozen_sizes(ls, key: str) -> List[int]:
    a, b = ls.branches
    if key == "w_in":
        return [a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim, a.heads * a.vdim, b.heads * b.dim, b.heads * b.dim,
                b.heads * b.vdim, b.heads * b.vdim, b.heads, b.heads]
    if key == "b_qkv":
        return [a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim]
    return [b.heads, b.heads]


def _load_zovozen_weights(rd, spec: ModelSpec, plan: StagePlan, device, dtype) -> StageWeights:
    w = StageWeights(spec, plan)
    get = lambda name: rd.get(name).to(device=device, dtype=dtype)
    w.embed, w.final_norm_w = get("embed"), get("final.norm")
    w.lm_head = w.embed
    for i in plan.layers:
        ls, l = spec.layer_specs[i], {}
        for k, names in _zovozen_layer_names(ls, f"l{i}.").items():
            if isinstance(names, tuple):
                l[k] = torch.cat([get(x) for x in names], dim=0)
            elif isinstance(names, list):
                l[k] = torch.stack([get(x) for x in names], dim=0)
            else:
                l[k] = get(names)
        for k, sizes in (("w_in", _zovozen_sizes(ls, "w_in")), ("b_qkv", _zovozen_sizes(ls, "b_qkv"))):
            if l[k].shape[0] != sum(sizes):
                raise ValueError(f"layer {i}: the mixer's projections have {l[k].shape[0]} rows, the config says {sum(sizes)}")
        if ls.moe is not None and l["w_router"].shape[0] != ls.moe.outputs:
            raise ValueError(f"layer {i}: the router has {l['w_router'].shape[0]} outputs, the config says {ls.moe.outputs}")
        w.layers.append(l)
    return w


def export_zovozen_state_dict(w: StageWeights) -> Dict[str, torch.Tensor]:
    """Logical -> checkpoint names (tests, `save` of random models)."""
    spec = w.spec
    sd = {"embed": w.embed, "final.norm": w.final_norm_w}
    for i, l in zip(w.plan.layers, w.layers):
        ls = spec.layer_specs[i]
        for k, names in _zovozen_layer_names(ls, f"l{i}.").items():
            if isinstance(names, tuple):
                for x, t in zip(names, torch.split(l[k], _zovozen_sizes(ls, k))):
                    sd[x] = t
            elif isinstance(names, list):
                for x, t in zip(names, l[k]):
                    sd[x] = t
            else:
                sd[names] = l[k]
    return {k: v.detach().clone().contiguous() for k, v in sd.items()}


def _random_zovozen_weights(spec: ModelSpec, plan: StagePlan, seed: int, device, dtype) -> StageWeights:
    """Random weights with which every mechanism matters: projections at 1 / sqrt(fan-in), biases, norm weights, head
    temperatures, mixing matrices, sinks and routing corrections of order one."""
    H, V = spec.hidden_size, spec.vocab_size
    w = StageWeights(spec, plan)
    rn = lambda name, shape, std: _randn(name, shape, seed, device, dtype, std=std)
    one = lambda name, shape, std: torch.ones(shape, device=device, dtype=dtype) + rn(name, shape, std)
    w.embed, w.final_norm_w = rn("embed", (V, H), 1.0), one("final.norm", (H,), 0.1)
    w.lm_head = w.embed
    for i in plan.layers:
        ls, p = spec.layer_specs[i], f"layers.{i}."
        a, b = ls.branches
        sizes = _zovozen_sizes(ls, "w_in")
        l: Dict[str, torch.Tensor] = {"ln1_w": one(p + "ln1_w", (H,), 0.2), "w_in": rn(p + "w_in", (sum(sizes), H), H ** -0.5)}
        l["b_qkv"] = rn(p + "b_qkv", (sum(sizes[:3]),), 0.3)
        l["q_norm_w"], l["k_norm_w"] = one(p + "q_norm_w", (sizes[0],), 0.2), one(p + "k_norm_w", (sizes[1],), 0.2)
        l["talk"] = torch.eye(a.heads, device=device, dtype=dtype) + rn(p + "talk", (a.heads, a.heads), 0.3)
        l["temp"], l["sink"] = one(p + "temp", (a.heads,), 0.3), rn(p + "sink", (a.heads,), 1.0)
        l["w_o"], l["b_o"] = rn(p + "w_o", (H, a.heads * a.vdim), (a.heads * a.vdim) ** -0.5), rn(p + "b_o", (H,), 0.2)
        l["b_if"] = rn(p + "b_if", (2 * b.heads,), 1.0)
        l["o_norm_w"], l["w_o_r"] = one(p + "o_norm_w", (b.heads * b.vdim,), 0.1), rn(p + "w_o_r", (H, b.heads * b.vdim), (b.heads * b.vdim) ** -0.5)
        if ls.has_ff:
            l["ln2_w"] = one(p + "ln2_w", (H,), 0.2)
        if ls.moe is not None:
            e = ls.moe
            l["w_router"], l["correction"] = rn(p + "w_router", (e.outputs, H), 2.0 * H ** -0.5), rn(p + "correction", (e.outputs,), 0.1)
            l["w_gate_e"], l["w_up_e"] = rn(p + "w_gate_e", (e.experts, e.ff, H), 1.5 * H ** -0.5), rn(p + "w_up_e", (e.experts, e.ff, H), 1.5 * H ** -0.5)
            l["w_down_e"] = rn(p + "w_down_e", (e.experts, H, e.ff), e.ff ** -0.5)
            if e.shared_ff:
                l["w_gate_s"], l["w_up_s"] = rn(p + "w_gate_s", (e.shared_ff, H), H ** -0.5), rn(p + "w_up_s", (e.shared_ff, H), H ** -0.5)
                l["w_down_s"] = rn(p + "w_down_s", (H, e.shared_ff), e.shared_ff ** -0.5)
        elif ls.ff:
            l["w_up"], l["b_up"] = rn(p + "w_up", (ls.ff, H), H ** -0.5), rn(p + "b_up", (ls.ff,), 0.2)
            l["w_down"], l["b_down"] = rn(p + "w_down", (H, ls.ff), ls.ff ** -0.5), rn(p + "b_down", (H,), 0.2)
        w.layers.append(l)
    return w


def _random_hybrid_weights(spec: ModelSpec, plan: StagePlan, seed: int, device, dtype) -> StageWeights:
    """Random weights of a hybrid stack, scaled so that activations stay of order one through any depth
    (projections at 1 / sqrt(fan-in), embedding at one) and every bias, convolution tap and gate matters."""
    if spec.family == "nufapel":
        return _random_nufapel_weights(spec, plan, seed, device, dtype)
    if spec.family == "tezesun":
        return _random_tezesun_weights(spec, plan, seed, device, dtype)
    if spec.family == "zovozen":
        return _random_zovozen_weights(spec, plan, seed, device, dtype)
    H, V = spec.hidden_size, spec.vocab_size
    w = StageWeights(spec, plan)
    rn = lambda name, shape, std: _randn(name, shape, seed, device, dtype, std=std)
    if plan.has_embed or plan.has_head:
        w.embed = rn("embed", (V, H), 1.0)
    for i in plan.layers:
        ls, p = spec.layer_specs[i], f"layers.{i}."
        qn, kn, vn, on = ls.qk_heads * ls.dim, ls.kv_heads * ls.dim, ls.v_heads * ls.vdim, ls.heads * ls.vdim
        l: Dict[str, torch.Tensor] = {"ln1_w": rn(p + "ln1_w", (H,), 0.1), "ln1b_w": rn(p + "ln1b_w", (H,), 0.1)}
        if ls.kind == "attention":
            l["w_qkv"] = rn(p + "w_qkv", (qn + kn + vn, H), H ** -0.5)
            l["b_qkv"] = rn(p + "b_qkv", (qn + kn + vn,), 0.3)
            l["vmix"] = torch.full((), 0.25 + 0.5 * ((i * 7919 + seed) % 10) / 10.0, device=device, dtype=dtype)
        else:
            l["w_in"] = rn(p + "w_in", (qn + kn + vn + on + 2 * ls.heads, H), H ** -0.5)
            l["conv_w"] = rn(p + "conv_w", (qn + kn + vn, ls.conv), 0.6)
            l["A_log"] = rn(p + "A_log", (ls.heads,), 0.5)
            l["dt_bias"] = rn(p + "dt_bias", (ls.heads,), 0.5)
            l["o_norm_w"] = torch.ones(ls.vdim, device=device, dtype=dtype) + rn(p + "o_norm_w", (ls.vdim,), 0.1)
        l["w_o"] = rn(p + "w_o", (H, on), on ** -0.5)
        if ls.ff:
            l["ln2_w"], l["ln2b_w"] = rn(p + "ln2_w", (H,), 0.1), rn(p + "ln2b_w", (H,), 0.1)
            l["w_gate"], l["b_gate"] = rn(p + "w_gate", (ls.ff, H), H ** -0.5), rn(p + "b_gate", (ls.ff,), 0.2)
            l["w_up"], l["b_up"] = rn(p + "w_up", (ls.ff, H), H ** -0.5), rn(p + "b_up", (ls.ff,), 0.2)
            l["w_down"], l["b_down"] = rn(p + "w_down", (H, ls.ff), ls.ff ** -0.5), rn(p + "b_down", (H,), 0.2)
        w.layers.append(l)
    if plan.has_head:
        w.final_norm_w = rn("final_norm_w", (H,), 0.1)
        w.lm_head = w.embed
    return w


def _load_hybrid_weights(rd, spec: ModelSpec, plan: StagePlan, device, dtype) -> StageWeights:
    if spec.family == "nufapel":
        return _load_nufapel_weights(rd, spec, plan, device, dtype)
    if spec.family == "tezesun":
        return _load_tezesun_weights(rd, spec, plan, device, dtype)
    if spec.family == "zovozen":
        return _load_zovozen_weights(rd, spec, plan, device, dtype)
    w = StageWeights(spec, plan)
    get = lambda name: rd.get(name).to(device=device, dtype=dtype)
    if plan.has_embed or plan.has_head:
        w.embed = get("embed")
    for i in plan.layers:
        ls, p = spec.layer_specs[i], f"l{i}."
        m = p + "mix."
        l = {"ln1_w": get(p + "norm1"), "ln1b_w": get(p + "norm1b"), "w_o": get(m + "o")}
        if ls.kind == "attention":
            l["w_qkv"] = torch.cat([get(m + x) for x in "qkv"], dim=0)
            l["b_qkv"] = torch.cat([get(m + x + ".b") for x in "qkv"], dim=0)
            l["vmix"] = get(m + "vmix").reshape(())
        else:
            l["w_in"] = torch.cat([get(m + x) for x in ("q", "k", "v", "g", "b", "a")], dim=0)
            l["conv_w"] = torch.cat([get(m + x + ".conv") for x in "qkv"], dim=0)
            l["A_log"], l["dt_bias"], l["o_norm_w"] = get(m + "A_log"), get(m + "dt_bias"), get(m + "norm")
        if ls.ff:
            f = p + "mlp."
            l.update({"ln2_w": get(p + "norm2"), "ln2b_w": get(p + "norm2b"),
                      "w_gate": get(f + "gate"), "b_gate": get(f + "gate.b"), "w_up": get(f + "up"), "b_up": get(f + "up.b"),
                      "w_down": get(f + "down"), "b_down": get(f + "down.b")})
        w.layers.append(l)
    if plan.has_head:
        w.final_norm_w = get("final.norm")
        w.lm_head = w.embed
    return w


def export_letarax_state_dict(w: StageWeights) -> Dict[str, torch.Tensor]:
    """Logical -> checkpoint names for a hybrid stack held by one stage (tests, `save` of random models)."""
    spec, sd = w.spec, {"embed": w.embed, "final.norm": w.final_norm_w}
    for i, l in zip(w.plan.layers, w.layers):
        ls, p = spec.layer_specs[i], f"l{i}."
        m = p + "mix."
        qn, kn, vn, on = ls.qk_heads * ls.dim, ls.kv_heads * ls.dim, ls.v_heads * ls.vdim, ls.heads * ls.vdim
        sd[p + "norm1"], sd[p + "norm1b"], sd[m + "o"] = l["ln1_w"], l["ln1b_w"], l["w_o"]
        if ls.kind == "attention":
            for x, t, b in zip("qkv", torch.split(l["w_qkv"], [qn, kn, vn]), torch.split(l["b_qkv"], [qn, kn, vn])):
                sd[m + x], sd[m + x + ".b"] = t, b
            sd[m + "vmix"] = l["vmix"]
        else:
            parts = torch.split(l["w_in"], [qn, kn, vn, on, ls.heads, ls.heads])
            for x, t in zip(("q", "k", "v", "g", "b", "a"), parts):
                sd[m + x] = t
            for x, t in zip("qkv", torch.split(l["conv_w"], [qn, kn, vn])):
                sd[m + x + ".conv"] = t
            sd[m + "A_log"], sd[m + "dt_bias"], sd[m + "norm"] = l["A_log"], l["dt_bias"], l["o_norm_w"]
        if ls.ff:
            f = p + "mlp."
            sd[p + "norm2"], sd[p + "norm2b"] = l["ln2_w"], l["ln2b_w"]
            for x in ("gate", "up", "down"):
                sd[f + x], sd[f + x + ".b"] = l["w_" + x], l["b_" + x]
    return {k: v.detach().clone().contiguous() for k, v in sd.items()}


def random_stage_weights(spec: ModelSpec, plan: StagePlan, seed: int = 0, device="cpu",
                         dtype=torch.float32) -> StageWeights:
    """Random-init weights of the given architecture for one stage."""
    if spec.is_hybrid:
        return _random_hybrid_weights(spec, plan, seed, device, dtype)
    H, I, V = spec.hidden_size, spec.intermediate_size, spec.vocab_size
    w = StageWeights(spec, plan)
    need_embed = plan.has_embed or (plan.has_head and spec.tie_embeddings)
    if need_embed:
        w.embed = _randn("embed", (V, H), seed, device, dtype)
    if plan.has_embed and spec.is_gpt2:
        w.pos_embed = _randn("pos_embed", (spec.max_position, H), seed, device, dtype, std=0.01)
    ones = lambda n: torch.ones(n, device=device, dtype=dtype)
    for i in plan.layers:
        p = f"layers.{i}."
        l: Dict[str, torch.Tensor] = {}
        attn, mlp = plan.has_attn(i), plan.has_mlp(i)       # a stage boundary may fall between a layer's two blocks
        if attn:
            l["ln1_w"] = ones(H) + _randn(p + "ln1_w", (H,), seed, device, dtype, std=0.05)
            l["w_qkv"] = _randn(p + "w_qkv", (spec.qkv_size, H), seed, device, dtype)
            l["w_o"] = _randn(p + "w_o", (H, spec.q_size), seed, device, dtype)
        if mlp:
            l["ln2_w"] = ones(H) + _randn(p + "ln2_w", (H,), seed, device, dtype, std=0.05)
        if spec.is_llama:
            # (as large as the projections' outputs, like the q/k/v biases of trained Qwen2 checkpoints: a numerics
            # test then fails when a path drops or misplaces a bias)
            if attn and spec.qkv_bias:
                l["b_qkv"] = _randn(p + "b_qkv", (spec.qkv_size,), seed, device, dtype, std=0.3)
            if attn and spec.o_bias:
                l["b_o"] = _randn(p + "b_o", (H,), seed, device, dtype, std=0.3)
            if mlp:
                l["w_gate"] = _randn(p + "w_gate", (I, H), seed, device, dtype)
                l["w_up"] = _randn(p + "w_up", (I, H), seed, device, dtype)
                l["w_down"] = _randn(p + "w_down", (H, I), seed, device, dtype)
        else:
            if attn:
                l["ln1_b"] = _randn(p + "ln1_b", (H,), seed, device, dtype)
                l["b_qkv"] = _randn(p + "b_qkv", (spec.qkv_size,), seed, device, dtype)
                l["b_o"] = _randn(p + "b_o", (H,), seed, device, dtype)
            if mlp:
                l["ln2_b"] = _randn(p + "ln2_b", (H,), seed, device, dtype)
                l["w_fc"] = _randn(p + "w_fc", (I, H), seed, device, dtype)
                l["b_fc"] = _randn(p + "b_fc", (I,), seed, device, dtype)
                l["w_down"] = _randn(p + "w_down", (H, I), seed, device, dtype)
                l["b_down"] = _randn(p + "b_down", (H,), seed, device, dtype)
        w.layers.append(l)
    if plan.has_head:
        w.final_norm_w = ones(H) + _randn("final_norm_w", (H,), seed, device, dtype, std=0.05)
        if spec.is_gpt2:
            w.final_norm_b = _randn("final_norm_b", (H,), seed, device, dtype)
        w.lm_head = w.embed if spec.tie_embeddings else _randn("lm_head", (V, H), seed, device, dtype)
    return w


# --------------------------------------------------------------------------------------
# Hugging Face checkpoint -> stage weights
# --------------------------------------------------------------------------------------

def stage_tensor_names(spec: ModelSpec, plan: StagePlan, available=None) -> List[str]:
    """The HF tensor names a stage needs (used by tests to prove nothing else is touched)."""
    names: List[str] = []
    if spec.is_llama:
        if plan.has_embed or (plan.has_head and spec.tie_embeddings):
            names.append("model.embed_tokens.weight")
        for i in plan.layers:
            p = f"model.layers.{i}."
            if plan.has_attn(i):
                names += [p + "input_layernorm.weight"] + [p + f"self_attn.{x}_proj.weight" for x in "qkvo"]
                names += [p + f"self_attn.{x}_proj.bias" for x in ("qkv" if spec.qkv_bias else "") + ("o" if spec.o_bias else "")]
            if plan.has_mlp(i):
                names += [p + "post_attention_layernorm.weight"] + [p + f"mlp.{x}_proj.weight" for x in ("gate", "up", "down")]
        if plan.has_head:
            names.append("model.norm.weight")
            if not spec.tie_embeddings:
                names.append("lm_head.weight")
    else:
        if plan.has_embed or plan.has_head:
            names.append("wte.weight")
        if plan.has_embed:
            names.append("wpe.weight")
        for i in plan.layers:
            p = f"h.{i}."
            for m in (("ln_1", "attn.c_attn", "attn.c_proj") if plan.has_attn(i) else ()) + \
                     (("ln_2", "mlp.c_fc", "mlp.c_proj") if plan.has_mlp(i) else ()):
                names += [p + m + ".weight", p + m + ".bias"]
        if plan.has_head:
            names += ["ln_f.weight", "ln_f.bias"]
    return names


def load_stage_weights(model_dir: str, spec: ModelSpec, plan: StagePlan, device="cpu",
                       dtype=torch.float32, reader: Optional[CheckpointReader] = None) -> StageWeights:
    """Read exactly this stage's tensors from a HF checkpoint directory."""
    rd = reader or CheckpointReader(model_dir)
    if spec.is_hybrid:
        w = _load_hybrid_weights(rd, spec, plan, device, dtype)
        if reader is None:
            rd.close()
        return w
    w = StageWeights(spec, plan)

    def get(name):
        t = rd.get(name)
        return t.to(device=device, dtype=dtype)

    if spec.is_llama:
        has_lm_head = "lm_head.weight" in rd
        tied = spec.tie_embeddings or not has_lm_head
        if plan.has_embed or (plan.has_head and tied):
            w.embed = get("model.embed_tokens.weight")
        for i in plan.layers:
            p = f"model.layers.{i}."
            l = {}
            if plan.has_attn(i):
                l.update({
                    "ln1_w": get(p + "input_layernorm.weight"),
                    "w_qkv": torch.cat([get(p + "self_attn.q_proj.weight"),
                                        get(p + "self_attn.k_proj.weight"),
                                        get(p + "self_attn.v_proj.weight")], dim=0),
                    "w_o": get(p + "self_attn.o_proj.weight")})
                if spec.qkv_bias:
                    l["b_qkv"] = torch.cat([get(p + f"self_attn.{x}_proj.bias") for x in "qkv"], dim=0)
                if spec.o_bias:
                    l["b_o"] = get(p + "self_attn.o_proj.bias")
            if plan.has_mlp(i):
                l.update({
                    "ln2_w": get(p + "post_attention_layernorm.weight"),
                    "w_gate": get(p + "mlp.gate_proj.weight"),
                    "w_up": get(p + "mlp.up_proj.weight"),
                    "w_down": get(p + "mlp.down_proj.weight")})
            w.layers.append(l)
        if plan.has_head:
            w.final_norm_w = get("model.norm.weight")
            w.lm_head = w.embed if tied else get("lm_head.weight")
    else:
        pre = "transformer." if "transformer.wte.weight" in rd else ""
        if plan.has_embed or plan.has_head:
            w.embed = get(pre + "wte.weight")
        if plan.has_embed:
            w.pos_embed = get(pre + "wpe.weight")
        for i in plan.layers:
            p = f"{pre}h.{i}."
            # Conv1D stores [in, out]; the engine wants [out, in]
            l = {}
            if plan.has_attn(i):
                l.update({
                    "ln1_w": get(p + "ln_1.weight"), "ln1_b": get(p + "ln_1.bias"),
                    "w_qkv": get(p + "attn.c_attn.weight").t().contiguous(), "b_qkv": get(p + "attn.c_attn.bias"),
                    "w_o": get(p + "attn.c_proj.weight").t().contiguous(), "b_o": get(p + "attn.c_proj.bias")})
            if plan.has_mlp(i):
                l.update({
                    "ln2_w": get(p + "ln_2.weight"), "ln2_b": get(p + "ln_2.bias"),
                    "w_fc": get(p + "mlp.c_fc.weight").t().contiguous(), "b_fc": get(p + "mlp.c_fc.bias"),
                    "w_down": get(p + "mlp.c_proj.weight").t().contiguous(), "b_down": get(p + "mlp.c_proj.bias")})
            w.layers.append(l)
        if plan.has_head:
            w.final_norm_w = get(pre + "ln_f.weight")
            w.final_norm_b = get(pre + "ln_f.bias")
            w.lm_head = w.embed
    if reader is None:
        rd.close()
    return w


def export_hf_state_dict(parts: List[StageWeights]) -> Dict[str, torch.Tensor]:
    """Inverse mapping (logical -> HF names) over all stages; used by tests to build HF models
    holding exactly the engine's random weights."""
    spec = parts[0].spec
    sd: Dict[str, torch.Tensor] = {}
    for w in parts:
        if spec.is_llama:
            if w.plan.has_embed:
                sd["model.embed_tokens.weight"] = w.embed
            for i, l in zip(w.plan.layers, w.layers):
                p = f"model.layers.{i}."
                if "w_qkv" in l:
                    q, k, v = torch.split(l["w_qkv"], [spec.q_size, spec.kv_size, spec.kv_size], dim=0)
                    sd[p + "input_layernorm.weight"] = l["ln1_w"]
                    sd[p + "self_attn.q_proj.weight"] = q
                    sd[p + "self_attn.k_proj.weight"] = k
                    sd[p + "self_attn.v_proj.weight"] = v
                    sd[p + "self_attn.o_proj.weight"] = l["w_o"]
                    if "b_qkv" in l:
                        for x, b in zip("qkv", torch.split(l["b_qkv"], [spec.q_size, spec.kv_size, spec.kv_size], dim=0)):
                            sd[p + f"self_attn.{x}_proj.bias"] = b
                    if "b_o" in l:
                        sd[p + "self_attn.o_proj.bias"] = l["b_o"]
                if "w_down" in l:
                    sd[p + "post_attention_layernorm.weight"] = l["ln2_w"]
                    sd[p + "mlp.gate_proj.weight"] = l["w_gate"]
                    sd[p + "mlp.up_proj.weight"] = l["w_up"]
                    sd[p + "mlp.down_proj.weight"] = l["w_down"]
            if w.plan.has_head:
                sd["model.norm.weight"] = w.final_norm_w
                if not spec.tie_embeddings:
                    sd["lm_head.weight"] = w.lm_head
        else:
            pre = "transformer."
            if w.plan.has_embed:
                sd[pre + "wte.weight"] = w.embed
                sd[pre + "wpe.weight"] = w.pos_embed
            for i, l in zip(w.plan.layers, w.layers):
                p = f"{pre}h.{i}."
                if "w_qkv" in l:
                    sd[p + "ln_1.weight"], sd[p + "ln_1.bias"] = l["ln1_w"], l["ln1_b"]
                    sd[p + "attn.c_attn.weight"], sd[p + "attn.c_attn.bias"] = l["w_qkv"].t(), l["b_qkv"]
                    sd[p + "attn.c_proj.weight"], sd[p + "attn.c_proj.bias"] = l["w_o"].t(), l["b_o"]
                if "w_down" in l:
                    sd[p + "ln_2.weight"], sd[p + "ln_2.bias"] = l["ln2_w"], l["ln2_b"]
                    sd[p + "mlp.c_fc.weight"], sd[p + "mlp.c_fc.bias"] = l["w_fc"].t(), l["b_fc"]
                    sd[p + "mlp.c_proj.weight"], sd[p + "mlp.c_proj.bias"] = l["w_down"].t(), l["b_down"]
            if w.plan.has_head:
                sd[pre + "ln_f.weight"], sd[pre + "ln_f.bias"] = w.final_norm_w, w.final_norm_b
    return {k: v.detach().clone().contiguous() for k, v in sd.items()}

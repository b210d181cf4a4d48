"""Pure-PyTorch pipeline-stage executor (the golden model and the no-GPU backend).

Implements exactly the stage interface of the GPU executor — ragged `StepBatch` in, hidden
states or logits out, with a per-sequence KV cache — using plain torch ops, so the scheduler,
transports, API and every pipeline-equivalence property are testable on CPU, and so the HIP
path has an independent model to be compared with.

What a stage computes is what the reference's `Worker.process` computes for its layer range
(Worker1.py:82-177: position ids, RoPE, the decoder-layer loop), plus the orchestrator's head
and tail on the first/last stage (orchestration.py:111 embedding, :140-141 final norm +
lm_head) — except that only new tokens are processed (KV cache) and only the rows that will
be sampled go through the final norm and lm_head.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..ops import reference as R
from ..runtime.batch import StepBatch
from ..runtime.sampler import filter_logits
from .partition import StagePlan
from .rope import build_rope_table
from .spec import ModelSpec
from .weights import StageWeights


class RefStage:
    backend = "torch"

    def __init__(self, spec: ModelSpec, plan: StagePlan, weights: StageWeights, dtype=torch.float32,
                 device="cpu", max_seq_len: Optional[int] = None):
        self.spec, self.plan = spec, plan
        self.dtype, self.device = dtype, torch.device(device)
        self.w = weights.to(device=self.device, dtype=dtype)
        self.max_seq_len = max_seq_len or min(spec.max_position, spec.sliding_window or spec.max_position)
        spec.check_context(self.max_seq_len)
        if spec.is_llama:
            self.cos, self.sin = build_rope_table(spec, self.max_seq_len, self.device)
        if spec.is_hybrid and not (plan.has_embed and plan.has_head):
            raise ValueError("a hybrid stack runs on one stage (its value mixing spans layers)")
        # slot -> per-layer [K, V] tensors of shape [len, Hkv, D]; a delta-rule layer of a hybrid stack keeps
        # [last conv inputs [taps-1, C], state [H, d, dv]] there instead
        self.cache: Dict[int, List[List[torch.Tensor]]] = {}

    # -- helpers --------------------------------------------------------------------------
    def _norm(self, x, w, b):
        if self.spec.is_llama:
            return R.rmsnorm(x, w, self.spec.norm_eps).to(self.dtype)
        return R.layernorm(x, w, b, self.spec.norm_eps).to(self.dtype)

    def _slot_cache(self, slot: int):
        c = self.cache.get(slot)
        if c is None:
            if self.spec.is_hybrid and self.spec.norm_kind == "dyt":
                # one entry per layer RUN (a repeated stretch of layers owns a cache / state per pass)
                c = [self._fresh_layer_state(self.spec.layer_specs[i]) for i, _ in self.spec.layer_runs()]
            elif self.spec.is_hybrid:
                c = [self._fresh_layer_state(self.spec.layer_specs[i]) for i in self.plan.layers]
                if self.spec.token_shift:           # every layer also carries the previous token's normed input
                    for st in c:
                        st.append(torch.zeros(self.spec.hidden_size, dtype=torch.float32, device=self.device))
            else:
                z = lambda: torch.zeros(0, self.spec.num_kv_heads, self.spec.head_dim, dtype=self.dtype, device=self.device)
                c = [[z(), z()] for _ in self.plan.layers]
            self.cache[slot] = c
        return c

    def _fresh_layer_state(self, ls):
        dev = self.device
        z32 = lambda *shape: torch.zeros(*shape, dtype=torch.float32, device=dev)
        if ls.kind == "parallel":
            return [self._fresh_layer_state(b) for b in ls.branches]
        if ls.kind == "general_delta":
            return [z32(ls.heads, ls.dim, ls.dim)]
        if ls.kind == "mlstm":
            return [z32(ls.heads, ls.dim, ls.vdim), z32(ls.heads, ls.dim), z32(ls.heads)]
        if ls.kind == "rglru":
            return [z32(max(ls.conv - 1, 0), ls.rec_width), z32(ls.rec_width)]
        if ls.kind == "latent_attention":
            return [torch.zeros(0, 1, ls.kv_rank, dtype=self.dtype, device=dev), torch.zeros(0, 1, ls.rot_dim, dtype=self.dtype, device=dev)]
        if ls.kind == "attention":
            return [torch.zeros(0, ls.kv_heads * ls.maps, ls.dim, dtype=self.dtype, device=dev),
                    torch.zeros(0, ls.kv_heads, ls.vdim, dtype=self.dtype, device=dev)]
        C = 2 * ls.kv_heads * ls.dim + ls.heads * ls.vdim
        return [torch.zeros(ls.conv - 1, C, dtype=torch.float32, device=dev),
                torch.zeros(ls.heads, ls.dim, ls.vdim, dtype=torch.float32, device=dev)]

    def release(self, slots: List[int]):
        for s in slots:
            self.cache.pop(s, None)

    # -- head / tail alone (the HTTP-compat orchestrator owns only these, as the reference's
    #    orchestrator does: orchestration.py:45-47) ---------------------------------------
    @torch.no_grad()
    def embed_tokens(self, ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        h = self.w.embed[ids.long()]
        if self.spec.is_gpt2:
            h = h + self.w.pos_embed[positions.long()]
        return h.to(self.dtype)

    @torch.no_grad()
    def head_logits(self, h_rows: torch.Tensor) -> torch.Tensor:
        hn = self._norm(h_rows.to(self.dtype), self.w.final_norm_w, self.w.final_norm_b)
        return R.gemm(hn, self.w.lm_head).float()

    # -- forward --------------------------------------------------------------------------
    # -- hybrid stacks: fp32 residual stream, a norm on both sides of every sublayer ------------------------------
    def _hybrid_layers(self, batch: StepBatch, h: torch.Tensor) -> torch.Tensor:
        """h [T, width] fp32 -> the residual stream after this stage's layers. Matrix products take their
        inputs in the compute dtype and accumulate in fp32; norms, scores, softmax, gates, decays and the
        recurrent state are fp32 whatever the dtype."""
        spec, dt, eps = self.spec, self.dtype, self.spec.norm_eps
        T = h.shape[0]
        lin = lambda x, w, b=None: R.gemm(x.to(dt), w, b, None, 1 if b is not None else 0)
        for slot, qlen, ctx in zip(batch.slots, batch.q_lens, batch.ctx_lens):
            if qlen > 0 and ctx == 0:
                self.cache.pop(slot, None)            # a sequence's first tokens: whatever the slot held before is void
        v_first = None
        for li, l in enumerate(self.w.layers):
            ls = spec.layer_specs[self.plan.layers[li]]
            xn = R.rmsnorm(h, l["ln1_w"], eps, unit_offset=True)
            H, G, d, dv = ls.heads, ls.kv_heads, ls.dim, ls.vdim
            mixed = torch.empty(T, H * dv, dtype=torch.float32, device=self.device)
            if ls.kind == "attention":
                qkv = lin(xn, l["w_qkv"], l["b_qkv"])
                q = qkv[:, :H * d].reshape(T, H, d).to(dt)
                k = qkv[:, H * d:(H + G) * d].reshape(T, G, d).to(dt)
                v = qkv[:, (H + G) * d:].reshape(T, G, dv)
                if ls.v_mix:
                    if v_first is None:
                        v_first = v
                    else:
                        lam = l["vmix"].float()
                        v = (1.0 - lam) * v + lam * v_first
                v = v.to(dt)
                t0 = 0
                for slot, qlen, ctx in zip(batch.slots, batch.q_lens, batch.ctx_lens):
                    if qlen == 0:
                        continue
                    kv = self._slot_cache(slot)[li]
                    assert kv[0].shape[0] >= ctx, f"slot {slot}: cache has {kv[0].shape[0]} tokens, step says {ctx}"
                    kv[0] = torch.cat([kv[0][:ctx], k[t0:t0 + qlen]])
                    kv[1] = torch.cat([kv[1][:ctx], v[t0:t0 + qlen]])
                    o = R.attention(q[t0:t0 + qlen], kv[0], kv[1], ctx, ls.scale, window=ls.window or 0, sink=ls.sink)
                    mixed[t0:t0 + qlen] = o.reshape(qlen, H * dv)
                    t0 += qlen
            else:
                qn, vn = G * d, H * dv
                z = lin(xn, l["w_in"])
                conv_in, gate = z[:, :2 * qn + vn], z[:, 2 * qn + vn:2 * qn + 2 * vn]
                beta = torch.sigmoid(z[:, 2 * qn + 2 * vn:2 * qn + 2 * vn + H])
                decay = torch.exp(-torch.exp(l["A_log"].float()) * torch.nn.functional.softplus(z[:, 2 * qn + 2 * vn + H:] + l["dt_bias"].float()))
                t0 = 0
                for slot, qlen, ctx in zip(batch.slots, batch.q_lens, batch.ctx_lens):
                    if qlen == 0:
                        continue
                    st = self._slot_cache(slot)[li]
                    y, st[0] = R.short_conv(conv_in[t0:t0 + qlen].to(dt), st[0], l["conv_w"])
                    y = torch.nn.functional.silu(y.to(dt).float())
                    qq = R.l2_unit(y[:, :qn].reshape(qlen, G, d)) * (d ** -0.5)
                    kk = R.l2_unit(y[:, qn:2 * qn].reshape(qlen, G, d))
                    o, st[1] = R.gated_delta_rule(qq, kk, y[:, 2 * qn:].reshape(qlen, H, dv), beta[t0:t0 + qlen],
                                                  decay[t0:t0 + qlen], st[1])
                    o = R.rmsnorm(o, l["o_norm_w"], eps) * torch.nn.functional.silu(gate[t0:t0 + qlen].to(dt).float()).reshape(qlen, H, dv)
                    mixed[t0:t0 + qlen] = o.reshape(qlen, H * dv)
                    t0 += qlen
            h = h + R.rmsnorm(lin(mixed, l["w_o"]), l["ln1b_w"], eps, unit_offset=True)
            if ls.ff:
                xn = R.rmsnorm(h, l["ln2_w"], eps, unit_offset=True)
                act = R.gelu_tanh(lin(xn, l["w_gate"], l["b_gate"]).to(dt).float()) * lin(xn, l["w_up"], l["b_up"]).to(dt).float()
                h = h + R.rmsnorm(lin(act, l["w_down"], l["b_down"]), l["ln2b_w"], eps, unit_offset=True)
        return h

    # -- hybrid stacks with dynamic-tanh pre-norms and gated residuals -------------------------------------------
    def _gated_layers(self, batch: StepBatch, h: torch.Tensor) -> torch.Tensor:
        """x <- x + sigmoid(W_g n + b_g) * f(n), n = dyt(x), for the mixer and the feed-forward of every layer run. Norms,
        scores, routers, gates of the recurrences, their states and the residual sum are fp32 whatever the dtype."""
        spec, dt, eps, w = self.spec, self.dtype, self.spec.norm_eps, self.w
        T = h.shape[0]
        F = torch.nn.functional
        lin = lambda x, m, b=None: R.gemm(x.to(dt), m, b, None, 1 if b is not None else 0)
        rnd = lambda x: x.to(dt).float()
        seqs = []
        t0 = 0
        for slot, qlen, ctx in zip(batch.slots, batch.q_lens, batch.ctx_lens):
            if qlen > 0 and ctx == 0:
                self.cache.pop(slot, None)            # a sequence's first tokens: whatever the slot held before is void
            if qlen > 0:
                seqs.append((slot, t0, qlen, ctx))
            t0 += qlen
        self.layer_outputs = []
        for ri, (li, pas) in enumerate(spec.layer_runs()):
            ls, l = spec.layer_specs[li], w.layers[li]
            if pas >= 0 and li == spec.loop[0]:
                h = h + w.loop_step[pas].float()
            xn = R.dyt(h, l["ln1_w"], l["ln1_b"], l["ln1_a"])
            z = lin(xn, l["w_in"])
            if ls.kind == "general_delta":
                H, d = ls.heads, ls.dim
                n = H * d
                r_, k_, v_, g_, a_, w1 = torch.split(z, [n] * 5 + [z.shape[1] - 5 * n], dim=1)
                dec = torch.exp(-math.exp(-0.5) * torch.sigmoid(lin(torch.tanh(rnd(w1)), l["w_w2"]) + l["w0"].float()))
                a_ = torch.sigmoid(a_ + l["b_a"].float())
                o = torch.empty(T, H, d, dtype=torch.float32, device=self.device)
                for slot, s0, qlen, ctx in seqs:
                    st, sl = self._slot_cache(slot)[ri], slice(s0, s0 + qlen)
                    hv = lambda x: x[sl].reshape(qlen, H, d)
                    o[sl], st[0] = R.general_delta_rule(hv(r_), hv(k_), hv(v_), hv(dec), hv(a_), st[0])
                mixed = (R.rmsnorm(o, torch.ones(d, device=self.device), eps).reshape(T, n) * l["o_norm_w"].float() * torch.sigmoid(g_))
                y = lin(mixed, l["w_o"])
            else:
                a, b = ls.branches
                sizes = [a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim, a.heads, b.heads * b.dim, b.heads * b.dim,
                         b.heads * b.vdim, b.heads * b.vdim, b.heads, b.heads]
                q, k, v, gl, rq, rk, rv, rg, ri_, rf_ = torch.split(z, sizes, dim=1)
                bias = R.distance_bias_table(l["rel"], a.bias_max, max(c + n_ for _, _, n_, c in seqs))
                left = torch.empty(T, a.heads, a.vdim, dtype=torch.float32, device=self.device)
                right = torch.empty(T, b.heads, b.vdim, dtype=torch.float32, device=self.device)
                li_ = b.gate_cap * torch.tanh((ri_ + l["b_if"][:b.heads].float()) / b.gate_cap)
                lf_ = F.logsigmoid(b.gate_cap * torch.tanh((rf_ + l["b_if"][b.heads:].float()) / b.gate_cap))
                for slot, s0, qlen, ctx in seqs:
                    sta, stb = self._slot_cache(slot)[ri]
                    sl = slice(s0, s0 + qlen)
                    assert sta[0].shape[0] >= ctx, f"slot {slot}: cache has {sta[0].shape[0]} tokens, step says {ctx}"
                    sta[0] = torch.cat([sta[0][:ctx], k[sl].reshape(qlen, a.kv_heads, a.dim).to(dt)])
                    sta[1] = torch.cat([sta[1][:ctx], v[sl].reshape(qlen, a.kv_heads, a.vdim).to(dt)])
                    left[sl] = R.attention(q[sl].reshape(qlen, a.heads, a.dim).to(dt), sta[0], sta[1], ctx, a.scale, sink=True,
                                           temp=l["temp"], dist_bias=bias, sink_logit=l["sink"])
                    right[sl], stb[0], stb[1], stb[2] = R.matrix_memory(
                        rq[sl].reshape(qlen, b.heads, b.dim) * b.scale, rk[sl].reshape(qlen, b.heads, b.dim),
                        rv[sl].reshape(qlen, b.heads, b.vdim), li_[sl], lf_[sl], stb[0], stb[1], stb[2])
                left = (left * torch.sigmoid(gl).unsqueeze(2)).reshape(T, -1)
                right = R.rmsnorm(right, torch.ones(b.vdim, device=self.device), eps).reshape(T, -1) * l["o_norm_w"].float() * torch.sigmoid(rg)
                y = 0.5 * (R.rmsnorm(lin(left, l["w_o"]), l["out_l"], eps) + R.rmsnorm(lin(right, l["w_o_r"]), l["out_r"], eps))
            h = h + torch.sigmoid(lin(xn, l["w_rg1"], l["b_rg1"])) * y
            if ls.has_ff:
                xn = R.dyt(h, l["ln2_w"], l["ln2_b"], l["ln2_a"])
                if ls.moe is None:
                    y = lin(rnd(R.gelu_erf(lin(xn, l["w_up"]))), l["w_down"])
                else:
                    e = ls.moe
                    idx, wts = R.moe_route(torch.sigmoid(lin(xn, l["w_router"])), e.top, e.groups, e.keep, e.scale)
                    y = torch.zeros_like(h)
                    for ex in range(e.experts):
                        rows, col = (idx == ex).nonzero(as_tuple=True)
                        if rows.numel() == 0:
                            continue
                        g = lin(xn[rows], l["w_gate_e"][ex]).clamp(max=e.limit)
                        u = lin(xn[rows], l["w_up_e"][ex]).clamp(min=-e.limit, max=e.limit)
                        y.index_add_(0, rows, lin(rnd(g * torch.sigmoid(1.702 * g) * (u + 1.0)), l["w_down_e"][ex]) * wts[rows, col].unsqueeze(1))
                h = h + torch.sigmoid(lin(xn, l["w_rg2"], l["b_rg2"])) * y
            self.layer_outputs.append(h)
        return h

    # -- hybrid stacks with parallel layers: one norm feeds the mixer and the feed-forward -------------------------
    def _parallel_layers(self, batch: StepBatch, h: torch.Tensor) -> torch.Tensor:
        """x <- x + ls1 * mixer(shifted(n)) + ls2 * ff(n), n = rms(x) w, for every layer. Norms, rotations, scores, the
        recurrence with its gates, and the residual sum are fp32 whatever the dtype."""
        from .rope import rope_table
        spec, dt, eps, w = self.spec, self.dtype, self.spec.norm_eps, self.w
        T, dev = h.shape[0], self.device
        F = torch.nn.functional
        lin = lambda x, m, b=None: R.gemm(x.to(dt), m, b, None, 1 if b is not None else 0)
        rnd = lambda x: x.to(dt).float()
        seqs, t0 = [], 0
        for slot, qlen, ctx in zip(batch.slots, batch.q_lens, batch.ctx_lens):
            if qlen > 0 and ctx == 0:
                self.cache.pop(slot, None)            # a sequence's first tokens: whatever the slot held before is void
            if qlen > 0:
                seqs.append((slot, t0, qlen, ctx))
            t0 += qlen
        pos = torch.tensor([c + i for c, q in zip(batch.ctx_lens, batch.q_lens) for i in range(q)], dtype=torch.long, device=dev)
        far = int(pos.max()) + 1 if T else 1
        self.layer_outputs = []
        for li, l in enumerate(w.layers):
            ls = spec.layer_specs[self.plan.layers[li]]
            n = R.rmsnorm(h, l["ln1_w"], eps)
            xm = torch.empty_like(n)
            for slot, s0, qlen, ctx in seqs:
                st = self._slot_cache(slot)[li]
                xm[s0:s0 + qlen], st[-1] = R.token_shift(n[s0:s0 + qlen], st[-1], l["shift"])
            z = lin(xm, l["w_in"], l.get("b_in"))
            if ls.rope_dims:
                cos, sin = rope_table(ls.rope_dims, ls.rope_base, ls.rope_scaling, far, dev)
            if ls.kind == "rglru":
                W = ls.rec_width
                y, xb = R.gelu_tanh(z[:, :W]), z[:, W:]
                mixed = torch.empty(T, W, dtype=torch.float32, device=dev)
                for slot, s0, qlen, ctx in seqs:
                    st, sl = self._slot_cache(slot)[li], slice(s0, s0 + qlen)
                    u, st[0] = R.short_conv(xb[sl], st[0], l["conv_w"])
                    u = u + l["conv_b"].float()
                    gr = torch.sigmoid(R.block_linear(u, l["w_ra"], l["b_ra"]))
                    gi = torch.sigmoid(R.block_linear(u, l["w_ri"], l["b_ri"]))
                    S, st[1] = R.rglru_scan(u, gr, gi, l["lam"], st[1])
                    mixed[sl] = S * y[sl]
            elif ls.kind == "attention":
                H, G, d, dv, M = ls.heads, ls.kv_heads, ls.dim, ls.vdim, ls.maps
                qn, kn, vn = H * M * d, G * M * d, G * dv
                q, k = z[:, :qn].reshape(T, H * M, d), z[:, qn:qn + kn].reshape(T, G * M, d)
                if ls.rope_dims:
                    q, k = R.rope_partial(q, cos, sin, pos, ls.rope_interleaved), R.rope_partial(k, cos, sin, pos, ls.rope_interleaved)
                v, gate = z[:, qn + kn:qn + kn + vn].reshape(T, G, dv), z[:, qn + kn + vn:]
                lam = torch.exp((l["lq1"].float() * l["lk1"].float()).sum()) - torch.exp((l["lq2"].float() * l["lk2"].float()).sum()) + ls.diff
                mixed = torch.empty(T, H, dv, dtype=torch.float32, device=dev)
                for slot, s0, qlen, ctx in seqs:
                    st, sl = self._slot_cache(slot)[li], slice(s0, s0 + qlen)
                    assert st[0].shape[0] >= ctx, f"slot {slot}: cache has {st[0].shape[0]} tokens, step says {ctx}"
                    st[0] = torch.cat([st[0][:ctx], k[sl].to(dt)])
                    st[1] = torch.cat([st[1][:ctx], v[sl].to(dt)])
                    maps = []
                    for mp in range(M):         # map mp of every head: its own queries and keys over the shared values
                        maps.append(R.attention(q[sl][:, mp::M], st[0][:, mp::M], st[1], ctx, ls.scale, window=ls.window or 0,
                                                keep_first=ls.keep_first, softcap=ls.softcap))
                    o = maps[0] - lam * maps[1] if M == 2 else maps[0]
                    mixed[sl] = R.rmsnorm(o, torch.ones(dv, device=dev), eps) * (1.0 - ls.diff) if M == 2 else o
                mixed = mixed.reshape(T, H * dv) * torch.sigmoid(gate)
            else:
                H, d, dr, dv, Rk = ls.heads, ls.dim, ls.rot_dim, ls.vdim, ls.kv_rank
                cq = R.rmsnorm(z[:, :ls.q_rank], l["dq_norm"], eps)
                q = lin(cq, l["w_uq"]).reshape(T, H, d + dr)
                c = R.rmsnorm(z[:, ls.q_rank:ls.q_rank + Rk], l["dkv_norm"], eps)
                kr = z[:, ls.q_rank + Rk:].reshape(T, 1, dr)
                if ls.rope_dims:
                    kr = R.rope_partial(kr, cos, sin, pos, ls.rope_interleaved)
                    q = torch.cat([q[..., :d], R.rope_partial(q[..., d:], cos, sin, pos, ls.rope_interleaved)], dim=-1)
                mixed = torch.empty(T, H, dv, dtype=torch.float32, device=dev)
                for slot, s0, qlen, ctx in seqs:
                    st, sl = self._slot_cache(slot)[li], slice(s0, s0 + qlen)
                    assert st[0].shape[0] >= ctx, f"slot {slot}: cache has {st[0].shape[0]} tokens, step says {ctx}"
                    st[0] = torch.cat([st[0][:ctx], c[sl].reshape(qlen, 1, Rk).to(dt)])
                    st[1] = torch.cat([st[1][:ctx], kr[sl].to(dt)])
                    n_all = st[0].shape[0]
                    ku = lin(st[0][:, 0], l["w_uk"]).reshape(n_all, H, d)
                    vv = lin(st[0][:, 0], l["w_uv"]).reshape(n_all, H, dv)
                    kk = torch.cat([ku, st[1].float().expand(n_all, H, dr)], dim=-1)
                    mixed[sl] = R.attention(q[sl], kk, vv, ctx, ls.scale)
                mixed = mixed.reshape(T, H * dv)
            add = lin(mixed, l["w_o"]) * l["ls1"].float()
            if ls.ff:
                act = R.xielu(lin(n, l["w_up"]), l["act"][0], l["act"][1])
                add = add + lin(rnd(act), l["w_down"]) * l["ls2"].float()
            h = h + add
            self.layer_outputs.append(h)
        return h

    # -- hybrid stacks whose sublayers read the stream itself, with RMS norms on their outputs only ------------------
    def _postnorm_layers(self, batch: StepBatch, h: torch.Tensor) -> torch.Tensor:
        """x <- x + norm1(a * left(x) + b * right(x)); x <- x + norm2(ff(x)) for every layer: attention (whole-projection
        q / k norms, partial rotation, unit values, head temperatures, mixed heads, chunked mask, learned sink, output gate)
        beside a matrix memory; dense squared-relu or routed feed-forward (softmax scores, corrected choice, identity and
        shared experts). Norms, rotations, scores, routers, gates of the recurrence, its state and the residual sum are fp32
        whatever the dtype."""
        from .rope import rope_table
        spec, dt, eps, w = self.spec, self.dtype, self.spec.norm_eps, self.w
        T, dev = h.shape[0], self.device
        F = torch.nn.functional
        lin = lambda x, m, b=None: R.gemm(x.to(dt), m, b, None, 1 if b is not None else 0)
        rnd = lambda x: x.to(dt).float()
        seqs, t0 = [], 0
        for slot, qlen, ctx in zip(batch.slots, batch.q_lens, batch.ctx_lens):
            if qlen > 0 and ctx == 0:
                self.cache.pop(slot, None)            # a sequence's first tokens: whatever the slot held before is void
            if qlen > 0:
                seqs.append((slot, t0, qlen, ctx))
            t0 += qlen
        pos = torch.tensor([c + i for c, q in zip(batch.ctx_lens, batch.q_lens) for i in range(q)], dtype=torch.long, device=dev)
        far = int(pos.max()) + 1 if T else 1
        ones = lambda n: torch.ones(n, device=dev)
        self.layer_outputs = []
        for li, l in enumerate(w.layers):
            ls = spec.layer_specs[self.plan.layers[li]]
            a, b = ls.branches
            sizes = [a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim, a.heads * a.vdim, b.heads * b.dim, b.heads * b.dim,
                     b.heads * b.vdim, b.heads * b.vdim, b.heads, b.heads]
            z = lin(h, l["w_in"])
            q, k, v, gl, rq, rk, rv, rg, ri_, rf_ = torch.split(z, sizes, dim=1)
            bq, bk, bv = torch.split(l["b_qkv"].float(), sizes[:3])
            q, k, v = q + bq, k + bk, v + bv
            if a.qk_norm:
                q, k = R.rmsnorm(q, l["q_norm_w"], eps), R.rmsnorm(k, l["k_norm_w"], eps)
            q, k, v = q.reshape(T, a.heads, a.dim), k.reshape(T, a.kv_heads, a.dim), v.reshape(T, a.kv_heads, a.vdim)
            if a.rope_dims:
                cos, sin = rope_table(a.rope_dims, a.rope_base, a.rope_scaling, far, dev)
                q, k = R.rope_partial(q, cos, sin, pos, a.rope_interleaved), R.rope_partial(k, cos, sin, pos, a.rope_interleaved)
            if a.v_norm:
                v = R.rmsnorm(v, ones(a.vdim), eps)
            left = torch.empty(T, a.heads, a.vdim, dtype=torch.float32, device=dev)
            right = torch.empty(T, b.heads, b.vdim, dtype=torch.float32, device=dev)
            li_ = b.gate_cap * torch.tanh((ri_ + l["b_if"][:b.heads].float()) / b.gate_cap)
            lf_ = F.logsigmoid(b.gate_cap * torch.tanh((rf_ + l["b_if"][b.heads:].float()) / b.gate_cap))
            for slot, s0, qlen, ctx in seqs:
                sta, stb = self._slot_cache(slot)[li]
                sl = slice(s0, s0 + qlen)
                assert sta[0].shape[0] >= ctx, f"slot {slot}: cache has {sta[0].shape[0]} tokens, step says {ctx}"
                sta[0] = torch.cat([sta[0][:ctx], k[sl].to(dt)])
                sta[1] = torch.cat([sta[1][:ctx], v[sl].to(dt)])
                left[sl] = R.attention(q[sl].to(dt), sta[0], sta[1], ctx, a.scale, sink=a.sink, temp=l["temp"] if a.head_temp else None,
                                       sink_logit=l["sink"] if a.sink_learned else None, chunk=a.chunk,
                                       head_mix=l["talk"] if a.head_mix else None)
                right[sl], stb[0], stb[1], stb[2] = R.matrix_memory(
                    rq[sl].reshape(qlen, b.heads, b.dim) * b.scale, rk[sl].reshape(qlen, b.heads, b.dim),
                    rv[sl].reshape(qlen, b.heads, b.vdim), li_[sl], lf_[sl], stb[0], stb[1], stb[2])
            left = left.reshape(T, -1) * torch.sigmoid(gl)
            right = R.rmsnorm(right, ones(b.vdim), eps).reshape(T, -1) * l["o_norm_w"].float() * torch.sigmoid(rg)
            y = ls.branch_scales[0] * lin(left, l["w_o"], l["b_o"]) + ls.branch_scales[1] * lin(right, l["w_o_r"])
            h = h + R.rmsnorm(y, l["ln1_w"], eps)
            if ls.has_ff:
                if ls.moe is None:
                    y = lin(rnd(torch.relu(lin(h, l["w_up"], l["b_up"])) ** 2), l["w_down"], l["b_down"])
                else:
                    e = ls.moe
                    glu = lambda x, g_, u_, d_: lin(rnd(F.silu(lin(x, g_)) * lin(x, u_)), d_)
                    idx, wts = R.moe_route(torch.softmax(lin(h, l["w_router"]), dim=-1), e.top, e.groups, e.keep, e.scale,
                                           correction=l["correction"], group_rank=e.group_rank, renorm=e.renorm)
                    y = torch.zeros_like(h)
                    for ex in range(e.outputs):
                        rows, col = (idx == ex).nonzero(as_tuple=True)
                        if rows.numel() == 0:
                            continue
                        out = h[rows] if ex >= e.experts else glu(h[rows], l["w_gate_e"][ex], l["w_up_e"][ex], l["w_down_e"][ex])
                        y.index_add_(0, rows, out * wts[rows, col].unsqueeze(1))
                    if e.shared_ff:
                        y = y + glu(h, l["w_gate_s"], l["w_up_s"], l["w_down_s"])
                h = h + R.rmsnorm(y, l["ln2_w"], eps)
            self.layer_outputs.append(h)
        return h

    def _forward_hybrid(self, batch: StepBatch, x: torch.Tensor) -> torch.Tensor:
        T = batch.num_tokens
        ids = torch.as_tensor(x).to(self.device).long().reshape(-1)
        assert ids.numel() == T, f"expected {T} token ids, got {ids.numel()}"
        if self.spec.post_norm:
            h = self._postnorm_layers(batch, self.w.embed[ids].float())
            self.last_hidden = h
            rows = self._out_rows(batch)
            if not rows:
                return torch.empty(0, self.spec.vocab_size, dtype=torch.float32, device=self.device)
            hn = R.rmsnorm(h[rows], self.w.final_norm_w, self.spec.norm_eps)
            return R.gemm(hn.to(self.dtype), self.w.lm_head).float()
        if self.spec.parallel_block:
            h = self._parallel_layers(batch, self.w.embed[ids].float())
            self.last_hidden = h
            rows = self._out_rows(batch)
            if not rows:
                return torch.empty(0, self.spec.vocab_size, dtype=torch.float32, device=self.device)
            hn = R.rmsnorm(h[rows], self.w.final_norm_w, self.spec.norm_eps)
            return R.gemm(hn.to(self.dtype), self.w.lm_head).float() * self.spec.logit_scale
        if self.spec.norm_kind == "dyt":
            pos = torch.tensor([c + i for c, q in zip(batch.ctx_lens, batch.q_lens) for i in range(q)], dtype=torch.long, device=self.device)
            h = self.w.embed[ids].float()
            if self.spec.learned_positions:
                h = h + self.w.pos_embed[pos].float()
            h = self._gated_layers(batch, h)
            self.last_hidden = h
            rows = self._out_rows(batch)
            if not rows:
                return torch.empty(0, self.spec.vocab_size, dtype=torch.float32, device=self.device)
            hn = R.dyt(h[rows], self.w.final_norm_w, self.w.final_norm_b, self.w.final_norm_a)
            z = R.gemm(hn.to(self.dtype), self.w.lm_head).float()
            cap = self.spec.logit_softcap
            return cap * torch.tanh(z / cap) if cap > 0 else z
        h = self._hybrid_layers(batch, self.w.embed[ids].float())
        self.last_hidden = h
        rows = self._out_rows(batch)
        if not rows:
            return torch.empty(0, self.spec.vocab_size, dtype=torch.float32, device=self.device)
        hn = R.rmsnorm(h[rows], self.w.final_norm_w, self.spec.norm_eps, unit_offset=True)
        return R.gemm(hn.to(self.dtype), self.w.lm_head).float()

    @staticmethod
    def _out_rows(batch: StepBatch) -> List[int]:
        """Token rows whose logits a step returns: the rows it asks scores for, else the last row of every sampled sequence."""
        if batch.score_rows is not None:
            return list(batch.score_rows)
        rows, t0 = [], 0
        for qlen, s in zip(batch.q_lens, batch.sample):
            if s and qlen > 0:
                rows.append(t0 + qlen - 1)
            t0 += qlen
        return rows

    @torch.no_grad()
    def forward(self, batch: StepBatch, x: torch.Tensor) -> torch.Tensor:
        spec = self.spec
        if spec.is_hybrid:
            return self._forward_hybrid(batch, x)
        T = batch.num_tokens
        positions = torch.tensor([c + i for c, q in zip(batch.ctx_lens, batch.q_lens) for i in range(q)],
                                 dtype=torch.long, device=self.device)
        if self.plan.has_embed:
            ids = x.to(self.device).long().reshape(-1)
            assert ids.numel() == T, f"expected {T} token ids, got {ids.numel()}"
            h = self.w.embed[ids]
            if spec.is_gpt2:
                h = h + self.w.pos_embed[positions]
            h = h.to(self.dtype)
        else:
            h = x.to(device=self.device, dtype=self.dtype).reshape(T, spec.hidden_size)
        Hq, Hkv, D = spec.num_heads, spec.num_kv_heads, spec.head_dim
        scale = D ** -0.5
        for li, l in enumerate(self.w.layers):
          if "w_qkv" in l:                 # (a stage boundary may fall between a layer's attention and MLP blocks)
            xn = self._norm(h, l["ln1_w"], l.get("ln1_b"))
            qkv = R.gemm(xn, l["w_qkv"], l.get("b_qkv"), None, 1 if "b_qkv" in l else 0).to(self.dtype)
            q = qkv[:, :Hq * D].reshape(T, Hq, D)
            k = qkv[:, Hq * D:(Hq + Hkv) * D].reshape(T, Hkv, D)
            v = qkv[:, (Hq + Hkv) * D:].reshape(T, Hkv, D)
            if spec.is_llama:
                q = R.rope(q, self.cos, self.sin, positions).to(self.dtype)
                k = R.rope(k, self.cos, self.sin, positions).to(self.dtype)
            attn = torch.empty(T, Hq * D, dtype=self.dtype, device=self.device)
            t0 = 0
            for slot, qlen, ctx in zip(batch.slots, batch.q_lens, batch.ctx_lens):
                if qlen == 0:
                    continue
                kv = self._slot_cache(slot)[li]
                if kv[0].shape[0] != ctx:
                    # a chunk may be re-sent after a failed step: keep exactly `ctx` cached tokens
                    assert kv[0].shape[0] >= ctx, f"slot {slot}: cache has {kv[0].shape[0]} tokens, step says {ctx}"
                    kv[0], kv[1] = kv[0][:ctx], kv[1][:ctx]
                kv[0] = torch.cat([kv[0], k[t0:t0 + qlen]])
                kv[1] = torch.cat([kv[1], v[t0:t0 + qlen]])
                o = R.attention(q[t0:t0 + qlen], kv[0], kv[1], ctx, scale)
                attn[t0:t0 + qlen] = o.reshape(qlen, Hq * D).to(self.dtype)
                t0 += qlen
            h = R.gemm(attn, l["w_o"], l.get("b_o"), h, 3 if "b_o" in l else 2).to(self.dtype)
          if "w_down" in l:
            xn = self._norm(h, l["ln2_w"], l.get("ln2_b"))
            if spec.is_llama:
                act = R.gemm(xn, torch.cat([l["w_gate"], l["w_up"]], 0), None, None, 4).to(self.dtype)
                h = R.gemm(act, l["w_down"], None, h, 2).to(self.dtype)
            else:
                act = R.gemm(xn, l["w_fc"], l["b_fc"], None, 5).to(self.dtype)
                h = R.gemm(act, l["w_down"], l["b_down"], h, 3).to(self.dtype)
        if not self.plan.has_head:
            return h
        # last stage: only the final position of each sequence that asks for a token (or the rows to be scored)
        rows = self._out_rows(batch)
        if not rows:
            return torch.empty(0, spec.vocab_size, dtype=torch.float32, device=self.device)
        hn = self._norm(h[rows], self.w.final_norm_w, self.w.final_norm_b)
        return R.gemm(hn, self.w.lm_head).float()

    # -- sampling -------------------------------------------------------------------------
    @torch.no_grad()
    def sample(self, batch: StepBatch, logits: torch.Tensor) -> torch.Tensor:
        """One token per sampled sequence, in batch order. int32 [num_samples]."""
        out, r = [], 0
        for i in range(batch.num_seqs):
            if not batch.sample[i] or batch.q_lens[i] == 0:
                continue
            z = logits[r].float().cpu()
            r += 1
            t = batch.temperature[i]
            if t <= 0.0:
                out.append(int(torch.argmax(z)))
                continue
            probs = filter_logits(z, t, batch.top_k[i], batch.top_p[i])
            g = torch.Generator()
            g.manual_seed((int(batch.seeds[i]) * 1000003 + int(batch.sample_steps[i])) & 0x7FFFFFFFFFFFFFFF)
            out.append(int(torch.multinomial(probs, 1, generator=g)))
        return torch.tensor(out, dtype=torch.int32)

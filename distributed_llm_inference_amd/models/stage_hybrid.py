"""MI355X executor for hybrid stacks: models whose layers are listed one by one (`ModelSpec.layer_specs`),
each with its own token mixer — windowed softmax attention with a sink over the paged cache, or a gated
delta-rule recurrence over a per-sequence state — a norm on both sides of every sublayer, and a residual
stream in fp32.

It is a `GpuStage`: the same step descriptors, metadata upload, block table, slots, scoring / sampling head,
fixed-shape decode states and hipGraph capture. What differs is what a layer runs:

    h (fp32) -> norm -> [ qkv GEMM -> value mixing + cache write -> windowed attention
                        | input GEMM -> short conv + silu -> unit q, k -> delta rule -> per-head norm * gate ]
             -> o GEMM -> post-norm + residual add + the next pre-norm (one kernel)
             -> [ gate/up GEMM with the gelu * up epilogue -> down GEMM -> post-norm + add + next pre-norm ]

and what a sequence owns: besides its cache blocks (attention layers), one slot of every recurrent layer's
state arrays, indexed by the step descriptor's slot number (the row of the block table). A sequence's first
tokens (context length 0) start from a zero state inside the kernels, so a slot is reused without clearing.

Stacks with dynamic-tanh pre-norms and gated residuals (`spec.norm_kind == "dyt"`) run the same way through
`_layers_gated`: per layer RUN (a stretch of layers may repeat with the same weights; every run owns its cache and state)

    h (fp32) -> dyt norm -> ONE input GEMM (all projections of the mixer and the residual gate)
             -> [ decay GEMM (low rank) -> generalised delta rule -> per-head norm * gate -> o GEMM
                | cache write -> attention with distance bias / head temperature / learned sink / head gate -> o GEMM
                  beside   matrix memory (exponential gates) -> per-head norm * gate -> o GEMM ]
             -> gated residual add (+ mean of the two RMS-normed branches) + the next norm (one kernel)
             -> [ up GEMM -> gelu -> down GEMM | router -> plan -> the experts' GEMMs over sorted rows -> weighted sum ]
             -> gated residual add + the next norm

Stacks with parallel layers (`spec.parallel_block`: one RMS norm feeds the mixer and the feed-forward, whose outputs are
scaled by learned vectors and added together) run through `_layers_par`: per layer

    n = rms(h) w (fp32 and the GEMMs' type)  -> token shift (blend with the previous token's n; the last n is the slot's state)
             -> ONE input GEMM (all projections of the mixer)
             -> [ causal conv -> block-diagonal gate GEMM -> gated linear recurrence * gelu(y)
                | rotation + cache write -> attention over two score maps per head, combined, normed, gated
                | latent norms -> query up-projection -> rotation + cache write of (latent | rotated key part)
                  -> per-head absorption of the key up-projection into the query -> attention over the latent rows
                  -> per-head value up-projection ]
             -> o GEMM;   up GEMM -> xIELU -> down GEMM (reads n itself)
             -> h += ls1 * mixer + ls2 * ff, the slot's carried n saved, and the next layer's n (one kernel)

Stacks that norm their sublayers' OUTPUTS only (`spec.post_norm`: the sublayers read the stream itself) run through
`_layers_post`: per layer

    x (fp32, and in the GEMMs' type) -> ONE input GEMM (all projections of both mixers, biases in the epilogue)
             -> [ q / k norms over the whole projection + rotation + unit values + the head mix folded into the query
                  + cache write (one kernel) -> attention with chunked mask, learned sink and output gate (steps with prompt
                  portions: plain queries, the mix applied to the finished score tiles)
                  beside   matrix memory (exponential gates) -> per-head norm * weight * gate ]
             -> ONE output GEMM over both branches' rows (the branch weights' ratio rides in the memory's norm weight)
             -> x += rms(a y) w, and x in the GEMMs' type (one kernel)
             -> [ up GEMM -> squared relu -> down GEMM
                | router + shared gate / up GEMM -> route -> plan -> the experts' GEMMs over sorted rows -> weighted sum with
                  the identity experts' share of x;  silu(gate) * up -> shared down GEMM ]
             -> x += rms(ff) w

Matrix products take bf16 operands (or fp32: `dtype="fp32"`, everything in true 32-bit) and accumulate in
fp32; norms, scores, softmax, value mixing, gates, decays and states are fp32 in both modes.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from types import SimpleNamespace
from typing import Dict, List, Optional

import torch

from ..ops import packing
from .partition import StagePlan
from .spec import LayerSpec, ModelSpec
from .stage_gpu import BLOCK, GpuStage
from .weights import StageWeights


@dataclass
class _HybridWork:
    """Activation workspaces of one step in flight (the eager path owns one, every decode micro-batch its own)."""
    h: torch.Tensor              # fp32 [T, H]   residual stream
    xn: torch.Tensor             # act  [T, H]   normalised input of the next GEMM
    z: torch.Tensor              # fp32 flat     output of a mixer's input projection (q|k|v, or q|k|v|gate|beta|decay)
    y: torch.Tensor              # fp32 flat     convolved q|k|v of a recurrent mixer
    o: torch.Tensor              # fp32 flat     raw read-out of a recurrent mixer
    mixed: torch.Tensor          # act  flat     mixer output ahead of the o projection
    yo: torch.Tensor             # fp32 [T, H]   sublayer output ahead of its post-norm
    act: torch.Tensor            # act  flat     gated feed-forward activation
    vfirst: torch.Tensor         # fp32 flat     values of the first value-mixing layer, for this step's tokens
    gu: torch.Tensor             # bf16 flat     gate | up pre-activations where the packed-weight GEMM produced them
    qkv16: torch.Tensor          # bf16 flat     fused q | k | v of the attention layers that run on the MFMA attention kernels
    ws: torch.Tensor             # fp32          split-K workspace of the packed-weight GEMMs (its last 4096 words: arrival counters)
    head_x: Optional[torch.Tensor]
    logits: Optional[torch.Tensor]
    cmax: Optional[torch.Tensor] = None
    guided: bool = False         # (the any-shape head GEMM leaves no chunk maxima: the sampler reads whole rows)


class HybridGpuStage(GpuStage):
    backend = "hip"

    def __init__(self, spec: ModelSpec, plan: StagePlan, weights: StageWeights, *, device="cuda", max_slots: int = 256,
                 max_seq_len: int = 2048, num_blocks: Optional[int] = None, max_tokens: int = 2048, max_batch: int = 64,
                 use_graphs: bool = True, kv_mem_fraction: float = 0.85, dtype: str = "bf16", decode_states: int = 1,
                 defer_kv: bool = False, graph_sizes: Optional[List[int]] = None):
        if not torch.cuda.is_available():
            raise RuntimeError("HybridGpuStage needs a GPU; use RefStage on CPU")
        if not spec.is_hybrid:
            raise ValueError("HybridGpuStage runs models described layer by layer")
        if not (plan.has_embed and plan.has_head):
            raise ValueError("a hybrid stack runs on one stage (its value mixing spans layers)")
        if dtype not in ("bf16", "fp32"):
            raise ValueError("hybrid stacks run in bf16 or fp32")
        self.kv8, self.wmode, self.w8 = False, dtype, False
        self.act_dtype = torch.float32 if dtype == "fp32" else torch.bfloat16
        self._init_limits(spec, plan, device, max_slots, max_seq_len, max_tokens, max_batch, use_graphs, graph_sizes)
        self.specs: List[LayerSpec] = [spec.layer_specs[i] for i in plan.layers]
        for i, ls in zip(plan.layers, self.specs):
            if max(ls.dim, ls.vdim) > 512:
                raise ValueError(f"layer {i}: head sizes up to 512 are supported")
            if ls.kind in ("delta", "rglru") and not 1 <= ls.conv <= 16:
                raise ValueError(f"layer {i}: 1 to 16 convolution taps are supported")
            if ls.kind == "latent_attention" and (ls.kv_rank + ls.rot_dim > 1024 or ls.kv_rank > 512):
                raise ValueError(f"layer {i}: latents up to 512 (with the rotated part up to 1024) are supported")
            if ls.kind == "attention" and ls.maps * ls.dim > 1024:
                raise ValueError(f"layer {i}: score maps of a head up to 1024 entries together are supported")
        for i, ls in zip(plan.layers, self.specs):
            for b in ls.branches or (ls,):
                if max(b.dim, b.vdim) > 512:
                    raise ValueError(f"layer {i}: head sizes up to 512 are supported")
        mixers = [ls for ls in self.specs if ls.kind == "attention" and ls.v_mix]
        if len({(ls.kv_heads, ls.vdim) for ls in mixers}) > 1:
            raise ValueError("value mixing needs the same key / value heads and value size in every layer that mixes")
        dev, at = self.device, self.act_dtype
        f32 = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        mat = lambda t: t.to(device=dev, dtype=at).contiguous()
        # Projections whose inner size is a multiple of 128 run on the library's packed-weight GEMMs (the weight-streaming
        # kernel up to 256 rows, the 256 x 256 tile kernel above), bf16 only; every other shape, and the fp32 mode, runs on
        # the any-shape kernel. DLIA_HYBRID_PACKED=0 keeps everything on the any-shape kernel (A/B).
        self._packed = dtype == "bf16" and os.environ.get("DLIA_HYBRID_PACKED", "1") != "0"
        self.decode_rows = 256
        self._shapes = []                        # (N, K, has_bias) of every packed GEMM, for the workspace
        # Attention layers whose keys and values have one size, 64 or 128, with up to 16 query heads per key / value head run
        # on the library's MFMA attention kernels (fragment-ordered cache, the windowed / sink instantiations), bf16 only;
        # other sizes, and the fp32 mode, on the any-size kernel. DLIA_HYBRID_MFMA_ATTN=0 keeps all on the any-size kernel (A/B).
        mfma_ok = dtype == "bf16" and os.environ.get("DLIA_HYBRID_MFMA_ATTN", "1") != "0"
        self.mfma_attn = [mfma_ok and ls.kind == "attention" and ls.dim == ls.vdim and ls.dim in (64, 128) and ls.group <= 16
                          for ls in self.specs]
        self._no_rope = {D: torch.zeros(1, D // 2, device=self.device) for D in (64, 128)}
        if spec.norm_kind == "dyt":
            # one cache / state per layer RUN
            self._attn_of_run = [spec.layer_specs[li].branches[0] if spec.layer_specs[li].kind == "parallel" else None for li, _ in spec.layer_runs()]
            self.mfma_attn = [mfma_ok and a is not None and a.dim == a.vdim and a.dim in (64, 128) and a.group <= 16 for a in self._attn_of_run]
        else:
            self._attn_of_run = [ls if ls.kind == "attention" else None for ls in self.specs]
        self.gated = spec.norm_kind == "dyt"
        self.par = spec.parallel_block
        self.post = spec.post_norm
        self.runs = spec.layer_runs()
        if self.post:
            self.mfma_attn = [False] * len(self.specs)
            self._attn_of_run = [ls.branches[0] for ls in self.specs]
            # attention on the matrix cores in bf16 where a head's query row (all key heads side by side when the head mix is
            # folded into it) is a multiple of 8; other sizes, and the fp32 mode, on the one-wave-per-(token, head) kernel.
            # DLIA_POST_TILE_ATTN=0: all on that (A/B)
            tile_ok = dtype == "bf16" and os.environ.get("DLIA_POST_TILE_ATTN", "1") != "0"
            for i, a in zip(plan.layers, self._attn_of_run):
                if self._query_row(a) > 1024:
                    raise ValueError(f"layer {i}: a head's query row of {self._query_row(a)} entries (key heads x key size, with mixed heads) is beyond 1024")
            self._tile = [tile_ok and self._query_row(a) % 8 == 0 and a.vdim <= 512 for a in self._attn_of_run]
            # steps with prompt portions: where the sizes allow, the mix is applied to the finished score tiles instead of
            # being carried by the query (plain-size score products). DLIA_POST_MIXED_ATTN=0: the query carries it always (A/B)
            direct_ok = os.environ.get("DLIA_POST_MIXED_ATTN", "1") != "0"
            self._direct = [direct_ok and tile and (a.head_mix or a.head_temp) and not a.window and
                            bool(self.K.mixed_attention_fits(a.heads, a.kv_heads, a.dim, a.vdim))
                            for a, tile in zip(self._attn_of_run, self._tile)]
            self._load_post(weights, f32, mat)
        if self.post:
            pass
        elif self.par:
            self.mfma_attn = [False] * len(self.specs)
            # attention layers whose sizes are multiples of 8 run on the matrix cores in bf16 (values key-contiguous in the
            # cache); other sizes, and the fp32 mode, on the one-wave-per-(token, head) kernel. DLIA_PAR_TILE_ATTN=0: all on that (A/B)
            tile_ok = dtype == "bf16" and os.environ.get("DLIA_PAR_TILE_ATTN", "1") != "0"
            def fits(ls):        # (sizes in whole 16-byte pieces, a query tile within a workgroup's LDS, accumulators within the registers)
                d, dv = self._score_dim(ls), ls.kv_rank if ls.kind == "latent_attention" else ls.vdim
                return d % 8 == 0 and ls.maps * d <= 1024 and dv <= (128 if ls.maps == 2 else 512)
            self._tile = [tile_ok and ls.kind != "rglru" and fits(ls) for ls in self.specs]
            self._load_par(weights, f32, mat)
        elif self.gated:
            self._load_gated(weights, f32, mat)
        else:
            self.embed = mat(weights.embed)
            self.lm_head = self.embed
            self.lm_head_p = None
            self.pos_embed = None
            self.final_norm_w = f32(weights.final_norm_w)
            self.vocab_pad = packing.padded_n(spec.vocab_size)
            self.layers: List[Dict[str, torch.Tensor]] = []
            for i, ls in enumerate(self.specs):
                l = weights.layers[i]
                p: Dict[str, torch.Tensor] = {"ln1_w": f32(l["ln1_w"]), "ln1b_w": f32(l["ln1b_w"])}
                self._matrix(p, "w_o", mat(l["w_o"]), None)
                if ls.kind == "attention":
                    self._matrix(p, "w_qkv", mat(l["w_qkv"]), f32(l["b_qkv"]))
                    p["vmix"] = f32(l["vmix"]).reshape(1)
                else:
                    self._matrix(p, "w_in", mat(l["w_in"]), None)
                    p["conv_w"] = f32(l["conv_w"])
                    p["A_log"], p["dt_bias"], p["o_norm_w"] = f32(l["A_log"]), f32(l["dt_bias"]), f32(l["o_norm_w"])
                if ls.ff:
                    # gate and up rows interleaved in 16-row tiles, so that one wave holds both for the same output
                    # columns; a width that is no multiple of 16 is padded with zero rows (their activations are zero
                    # and meet zero columns of the down projection)
                    pad = (-ls.ff) % 16
                    padr = lambda t: torch.cat([t, t.new_zeros(pad, *t.shape[1:])]) if pad else t
                    p["ln2_w"], p["ln2b_w"] = f32(l["ln2_w"]), f32(l["ln2b_w"])
                    if self._packed and spec.hidden_size % 128 == 0 and ls.ff % 8 == 0:
                        # gate rows, then up rows, through the packed-weight GEMM; the gate is applied by a kernel of its own
                        self._matrix(p, "w_gu", torch.cat([mat(l["w_gate"]), mat(l["w_up"])]), torch.cat([f32(l["b_gate"]), f32(l["b_up"])]))
                        p["ff_cols"] = ls.ff
                    else:
                        p["w_gu"] = packing.interleave_gate_up(padr(mat(l["w_gate"])), padr(mat(l["w_up"]))).contiguous()
                        p["b_gu"] = packing.interleave_gate_up(padr(f32(l["b_gate"])).unsqueeze(1), padr(f32(l["b_up"])).unsqueeze(1)).reshape(-1).contiguous()
                        p["ff_cols"] = ls.ff + pad
                    wd = mat(l["w_down"])
                    if "w_gu_p" not in p and pad:
                        wd = torch.cat([wd, wd.new_zeros(wd.shape[0], pad)], dim=1).contiguous()
                    self._matrix(p, "w_down", wd, f32(l["b_down"]))
                self.layers.append(p)
                weights.layers[i] = {}
            if self._packed and spec.hidden_size % 128 == 0:
                self.lm_head_p = packing.pack_weight(self.embed)
                self._shapes.append((self.vocab_pad, spec.hidden_size, False))
        self._ws_floats = self._packed_ws_floats()
        self.keep_layer_outputs = False          # debugging aid: eager steps append the residual stream after every layer
        self.layer_outputs: List[torch.Tensor] = []
        self.wk0 = self._new_work(self.max_tokens)
        self._init_step_state(kv_mem_fraction, decode_states)
        # recurrent state, one slot per row of the block table (the null slot included: padding rows land there)
        self.rec: List[Optional[tuple]] = []
        for ls in (self.specs if self.par else []):
            # every layer: the previous token's normed input [slots + 1, H]; a recurrent unit also its convolution's last
            # inputs and its state, one number per channel
            st = (torch.zeros(max_slots + 1, spec.hidden_size, device=dev),)
            if ls.kind == "rglru":
                st += (torch.zeros(max_slots + 1, max(ls.conv - 1, 1), ls.rec_width, device=dev), torch.zeros(max_slots + 1, ls.rec_width, device=dev))
            self.rec.append(st)
        for ls in (self.specs if self.post else []):
            # the matrix memory's state (its normaliser as one more column) and running maxima
            b = ls.branches[1]
            self.rec.append((torch.zeros(max_slots + 1, b.heads, b.dim, b.vdim + 1, device=dev),
                             torch.zeros(max_slots + 1, b.heads, 128, device=dev)))
        for ls in ([spec.layer_specs[li] for li, _ in self.runs] if self.gated else []):
            if ls.kind == "general_delta":
                self.rec.append((torch.zeros(max_slots + 1, ls.heads, ls.dim, ls.dim, device=dev),))
            else:
                b = ls.branches[1]
                self.rec.append((torch.zeros(max_slots + 1, b.heads, b.dim, b.vdim + 1, device=dev),
                                 torch.zeros(max_slots + 1, b.heads, 128, device=dev)))
        for ls in ([] if (self.gated or self.par or self.post) else self.specs):
            if ls.kind == "delta":
                C = 2 * ls.kv_heads * ls.dim + ls.heads * ls.vdim
                self.rec.append((torch.zeros(max_slots + 1, max(ls.conv - 1, 1), C, device=dev),
                                 torch.zeros(max_slots + 1, ls.heads, ls.dim, ls.vdim, device=dev)))
            else:
                self.rec.append(None)
        if not defer_kv:
            self.allocate_kv(num_blocks if num_blocks is not None else self.kv_budget_blocks())

    # ---- matrices: packed for the library's tuned GEMMs where the shape allows, row-major otherwise --------------
    def _matrix(self, p: Dict[str, torch.Tensor], name: str, w: torch.Tensor, bias: Optional[torch.Tensor]):
        """Stores W [N, K] (+ fp32 bias) under `name`: as the packed image `name_p` (N padded to a multiple of 4 with
        zero rows: `name_n`; bias in bf16, which a bf16 checkpoint's bias is anyway) when K is a multiple of 128, as the
        row-major matrix for the any-shape kernel otherwise."""
        N, K = w.shape
        if self._packed and K % 128 == 0:
            n4 = (N + 3) // 4 * 4
            if n4 != N:
                w = torch.cat([w, w.new_zeros(n4 - N, K)])
                bias = torch.cat([bias, bias.new_zeros(n4 - N)]) if bias is not None else None
            p[name + "_p"], p[name + "_n"] = packing.pack_weight(w.contiguous()), n4
            if bias is not None:
                p[name + "_b"] = bias.to(torch.bfloat16).contiguous()
            self._shapes.append((n4, K, bias is not None))
        else:
            p[name] = w
            if bias is not None:
                p["b_" + name[2:]] = bias

    def _cols(self, p, name: str) -> int:
        """Output columns of the projection stored under `name` (the padded count when it is packed)."""
        return p[name + "_n"] if name + "_p" in p else p[name].shape[0]

    def _mm(self, wk, out: torch.Tensor, x: torch.Tensor, p, name: str):
        """out = x . W^T (+ bias) for the projection stored under `name`."""
        wp = p.get(name + "_p")
        if wp is None:
            self.K.gemm_any(out, x, p[name], p.get("b_" + name[2:]), 0)
            return
        b = p.get(name + "_b")
        # more than 256 rows: the tile kernel, spread over the whole chip when a shape has few tiles
        self.K.gemm(out, x, wp, b, None, wk.ws, p[name + "_n"], 1 if b is not None else 0, 256 if x.shape[0] > self.decode_rows else 0, 0)

    def _packed_ws_floats(self) -> int:
        need = 1
        for (n_, k_, hb) in self._shapes:
            for m_ in range(1, self.decode_rows + 1):
                sk = int(self.K.gemm_config(m_, n_, k_, 1 if hb else 0, True)[1])
                if sk > 1:
                    need = max(need, sk * m_ * n_)
        return need

    # ---- workspaces ---------------------------------------------------------------------------------------
    def _new_work(self, rows: int):
        if self.post:
            return self._new_work_post(rows)
        if self.par:
            return self._new_work_par(rows)
        if self.gated:
            return self._new_work_gated(rows)
        s, dev, at = self.spec, self.device, self.act_dtype
        z = lambda n, dt=torch.float32: torch.zeros(max(int(n), 1), device=dev, dtype=dt)
        B = min(rows, self.max_batch)
        H = s.hidden_size
        zc = yc = oc = mc = ac = vc = 1
        for ls in self.specs:
            qn, kn, vn, on = ls.qk_heads * ls.dim, ls.kv_heads * ls.dim, ls.v_heads * ls.vdim, ls.heads * ls.vdim
            mc, ac = max(mc, on), max(ac, (ls.ff + 15) // 16 * 16)
            if ls.kind == "attention":
                zc = max(zc, qn + kn + vn + 3)
                vc = max(vc, vn if ls.v_mix else 1)
            else:
                zc, yc, oc = max(zc, qn + kn + vn + on + 2 * ls.heads + 3), max(yc, qn + kn + vn), max(oc, on)
        ws_floats = self._ws_floats
        if self._packed and rows > self.decode_rows:
            for m_ in {rows, min(rows, 512), min(rows, 1024)}:
                if m_ > self.decode_rows:
                    ws_floats = max([ws_floats] + [int(self.K.gemm_ws_floats(m_, n_, k_)) for n_, k_, _ in self._shapes])
        guc = max([2 * ls.ff for ls in self.specs if ls.ff] + [1]) if self._packed else 1
        qc = max([(ls.heads + 2 * ls.kv_heads) * ls.dim for ls, fast in zip(self.specs, self.mfma_attn) if fast] + [1])
        return _HybridWork(
            h=torch.zeros(rows, H, device=dev), xn=torch.zeros(rows, H, device=dev, dtype=at), z=z(rows * zc), y=z(rows * yc),
            o=z(rows * oc), mixed=z(rows * mc, at), yo=torch.zeros(rows, H, device=dev), act=z(rows * ac, at),
            vfirst=z(rows * vc), gu=z(rows * guc, torch.bfloat16), qkv16=z(rows * qc, torch.bfloat16), ws=z(ws_floats + 4096), head_x=torch.zeros(B, H, device=dev, dtype=at),
            logits=torch.zeros(B, self.vocab_pad, device=dev))

    # ---- cache and state sizing -------------------------------------------------------------------------
    def kv_block_bytes(self) -> int:
        e = 4 if self.act_dtype == torch.float32 else 2
        if self.par:
            return max(1, sum(BLOCK * e * sum(self._par_rows(li)) for li, ls in enumerate(self.specs) if ls.kind != "rglru"))
        return max(1, sum(ls.kv_heads * BLOCK * (ls.dim + ls.vdim) * e for ls in self._attn_of_run if ls is not None))

    def _decode_state_bytes(self) -> int:
        n = 0
        if self.gated or self.par or self.post:
            per_row = sum(t.numel() * t.element_size() for t in vars(self.wk0).values() if torch.is_tensor(t)) // self.max_tokens
            return sum(B * (per_row + 4 * self.vocab_pad) for B in self.graph_sizes)
        for B in self.graph_sizes:
            w = self.wk0
            per_row = sum(t.numel() * t.element_size() for t in (w.h, w.xn, w.z, w.y, w.o, w.mixed, w.yo, w.act, w.vfirst)) // self.max_tokens
            n += B * (per_row + 4 * self.vocab_pad + 4 * self.spec.hidden_size)
        return n

    def allocate_kv(self, num_blocks: int):
        dev, at = self.device, self.act_dtype
        self.num_blocks = int(num_blocks)
        if self.post:
            # keys: with the head mix folded into the query every head reads ALL key heads, so a token's keys are one row;
            # values per key / value head, key-contiguous where the matrix-core kernel reads them
            self.kv = []
            for a, p, tile in zip(self._attn_of_run, self.layers, self._tile):
                G, gk = a.kv_heads, 1 if p["mix"] is not None else a.kv_heads
                kc = torch.zeros(self.num_blocks, gk, BLOCK, G * a.dim // gk, device=dev, dtype=at)
                vc = torch.zeros(self.num_blocks, G, a.vdim, BLOCK, device=dev, dtype=at) if tile else \
                    torch.zeros(self.num_blocks, G, BLOCK, a.vdim, device=dev, dtype=at)
                self.kv.append((kc, vc))
            return
        if self.par:
            # attention: key rows hold a head's score maps side by side, value rows apart; latent attention: ONE row per token,
            # the normed latent followed by the rotated key part (the values are the row's first entries)
            self.kv = []
            for li, ls in enumerate(self.specs):
                if ls.kind == "rglru":
                    self.kv.append(None)
                    continue
                kr, vr = self._par_rows(li)
                G = ls.kv_heads
                kc = torch.zeros(self.num_blocks, G, BLOCK, kr // G, device=dev, dtype=at)
                if self._tile[li]:        # values key-contiguous: [block][head][entry][32 tokens]
                    vc = torch.zeros(self.num_blocks, G, vr // G, BLOCK, device=dev, dtype=at)
                else:
                    vc = torch.zeros(self.num_blocks, G, BLOCK, vr // G, device=dev, dtype=at) if vr else kc
                self.kv.append((kc, vc))
            return
        # zero-filled: a row that was never written must hold finite values
        # (a layer on the MFMA attention kernels keeps K and V slabs of a block side by side, in fragment order)
        self.kv = [None if ls is None else
                   torch.zeros(self.num_blocks, ls.kv_heads, 2, BLOCK * ls.dim, device=dev, dtype=at) if fast else
                   (torch.zeros(self.num_blocks, ls.kv_heads, BLOCK, ls.dim, device=dev, dtype=at),
                    torch.zeros(self.num_blocks, ls.kv_heads, BLOCK, ls.vdim, device=dev, dtype=at))
                   for ls, fast in zip(self._attn_of_run, self.mfma_attn)]

    def _pick_splits(self, B: int, max_ctx: int) -> int:
        return 1

    def _capture(self, st):
        """Capturing a step runs it once for real beforehand (first-use initialisation must not happen under
        capture). A cache write of that run is harmless: the replay writes the same row again. A recurrent state is
        not idempotent: the same token applied twice is a different state. So the rows are parked on the null slot
        for the run and the capture (kernels read the slots from the static buffer at replay time, not now)."""
        saved = st.slots.clone()
        st.slots.fill_(self.null_slot)
        try:
            super()._capture(st)
        finally:
            st.slots.copy_(saved)

    # ---- the layer stack ----------------------------------------------------------------------------------
    def _embed_rows(self, wk, T: int, ids, pos):
        if self.pos_embed is not None:
            self.K.embed_pos32(wk.h[:T], ids, pos, self.embed, self.pos_embed)
        else:
            self.K.embed32(wk.h[:T], ids, self.embed)

    def _layers(self, wk: _HybridWork, T: int, B: int, tok_pos, tok_seq, q_start, ctx, slots, max_q: int, splits: int,
                alone: bool = False, lead_decode: int = 0):
        if self.post:
            return self._layers_post(wk, T, B, tok_pos, tok_seq, q_start, ctx, slots, max_q)
        if self.par:
            return self._layers_par(wk, T, B, tok_pos, tok_seq, q_start, ctx, slots, max_q)
        if self.gated:
            return self._layers_gated(wk, T, B, tok_pos, tok_seq, q_start, ctx, slots, max_q, lead_decode)
        K, eps = self.K, self.spec.norm_eps
        h, xn, yo = wk.h[:T], wk.xn[:T], wk.yo[:T]
        view = lambda buf, cols: buf[:T * cols].view(T, cols)
        keep = self.keep_layer_outputs and not torch.cuda.is_current_stream_capturing()
        if keep:
            self.layer_outputs = []
        K.norm32(xn, h, None, None, self.layers[0]["ln1_w"], None, eps, 1.0)
        seen_mix = False
        n_layers = len(self.layers)
        for li, (ls, p) in enumerate(zip(self.specs, self.layers)):
            Hh, G, d, dv = ls.heads, ls.kv_heads, ls.dim, ls.vdim
            mixed = view(wk.mixed, Hh * dv)
            if ls.kind == "attention" and self.mfma_attn[li]:
                qkv = view(wk.qkv16, (Hh + 2 * G) * d)
                self._mm(wk, qkv, xn, p, "w_qkv")
                mix = 0 if not ls.v_mix else (2 if seen_mix else 1)
                seen_mix = seen_mix or ls.v_mix
                if mix:
                    K.value_mix(qkv, wk.vfirst, p["vmix"] if mix == 2 else None, mix, (Hh + G) * d, G * d)
                K.rope_kvwrite(qkv, None, 1, None, self.kv[li], self._no_rope[d], self._no_rope[d], tok_pos, tok_seq,
                               self.block_table, Hh, G, d, False)
                win = ls.window or 0
                if 0 < lead_decode < B and max_q > 1:
                    # single tokens riding in front of prompt portions: the decode-shaped kernel for them, the prefill-shaped for the rest
                    n = lead_decode
                    K.paged_attention_window(mixed, qkv, self.kv[li], q_start[:n + 1], ctx[:n], self.block_table, slots[:n], None,
                                             1, Hh, G, d, ls.scale, 1, win, ls.sink)
                    K.paged_attention_window(mixed, qkv, self.kv[li], q_start[n:], ctx[n:], self.block_table, slots[n:], None,
                                             max_q, Hh, G, d, ls.scale, 1, win, ls.sink)
                else:
                    K.paged_attention_window(mixed, qkv, self.kv[li], q_start, ctx, self.block_table, slots, None, max_q, Hh, G, d,
                                             ls.scale, 1, win, ls.sink)
            elif ls.kind == "attention":
                z = view(wk.z, self._cols(p, "w_qkv"))
                self._mm(wk, z, xn, p, "w_qkv")
                mix = 0 if not ls.v_mix else (2 if seen_mix else 1)
                seen_mix = seen_mix or ls.v_mix
                kc, vc = self.kv[li]
                z = z[:, :(Hh + G) * d + G * dv]
                K.kv_store(z, wk.vfirst if mix else None, p["vmix"] if mix == 2 else None, mix, kc, vc, tok_pos, tok_seq,
                           self.block_table, G, d, dv, Hh * d)
                K.window_attention(mixed, z, kc, vc, tok_pos, tok_seq, self.block_table, Hh, G, d, dv, ls.scale,
                                   ls.window or 0, ls.sink)
            else:
                qn, vn = G * d, Hh * dv
                C = 2 * qn + vn
                z = view(wk.z, self._cols(p, "w_in"))
                y, o = view(wk.y, C), view(wk.o, vn)
                carry, state = self.rec[li]
                self._mm(wk, z, xn, p, "w_in")
                K.short_conv(y, z, carry, p["conv_w"], q_start, ctx, slots, max_q)
                K.unit_heads(y[:, :2 * qn], 2 * G, d, G, d ** -0.5, 1e-6)
                K.delta_rule(o, y, z, state, p["A_log"], p["dt_bias"], q_start, ctx, slots, G, Hh, d, dv, C + vn, C + vn + Hh, max_q)
                K.gated_headnorm(mixed, o, z[:, C:C + vn], p["o_norm_w"], Hh, dv, eps)
            self._mm(wk, yo, mixed, p, "w_o")
            nxt = self.layers[li + 1]["ln1_w"] if li + 1 < n_layers else None
            after_mixer = p["ln2_w"] if ls.ff else nxt
            K.norm32(xn if after_mixer is not None else None, h, yo, p["ln1b_w"], after_mixer, None, eps, 1.0)
            if ls.ff:
                act = view(wk.act, p["ff_cols"])
                if "w_gu_p" in p:
                    gu = view(wk.gu, 2 * ls.ff)
                    self._mm(wk, gu, xn, p, "w_gu")
                    K.gated_gelu(act, gu)
                else:
                    K.gemm_any(act, xn, p["w_gu"], p["b_gu"], 1)
                self._mm(wk, yo, act, p, "w_down")
                K.norm32(xn if nxt is not None else None, h, yo, p["ln2b_w"], nxt, None, eps, 1.0)
            if keep:
                self.layer_outputs.append(h.clone())
        return None

    # ---- stacks with dynamic-tanh norms and gated residuals -------------------------------------------------------
    def _load_gated(self, weights: StageWeights, f32, mat):
        """Device weights of a gated stack. Everything that reads a sublayer's input is ONE matrix: the mixer's projections and
        the residual gate (mixer), the up projection or the router and the residual gate (feed-forward). Biases stay apart and
        are added in fp32 by the kernels that consume the projections."""
        from ..ops import reference as R
        spec, dev = self.spec, self.device
        self.embed, self.pos_embed = mat(weights.embed), mat(weights.pos_embed) if spec.learned_positions else None
        self.lm_head = mat(weights.lm_head)
        self.lm_head_p = None
        self.final_norm_w, self.final_norm_b = f32(weights.final_norm_w), f32(weights.final_norm_b)
        self.final_norm_a = float(weights.final_norm_a)
        self.loop_step = f32(weights.loop_step) if spec.loop else None
        self.vocab_pad = packing.padded_n(spec.vocab_size)
        self.layers = []
        for i, ls in enumerate(self.specs):
            l = weights.layers[i]
            p = {k: f32(l[k]) for k in ("ln1_w", "ln1_b", "b_rg1", "o_norm_w")}
            p["ln1_a"] = float(l["ln1_a"])
            w_in = mat(l["w_in"])
            p["fast"] = False
            if ls.kind == "parallel":
                a = ls.branches[0]
                run = [ri for ri, (li, _) in enumerate(self.runs) if li == i][0]
                if self.mfma_attn[run]:
                    # q | k | v of the attention leave through a GEMM of their own, in bf16, for the MFMA attention kernels
                    c = (a.heads + a.kv_heads) * a.dim + a.kv_heads * a.vdim
                    self._matrix(p, "w_qkv", w_in[:c].contiguous(), None)
                    w_in, p["fast"] = w_in[c:], True
            self._matrix(p, "w_in", torch.cat([w_in, mat(l["w_rg1"])]), None)
            self._matrix(p, "w_o", mat(l["w_o"]), None)
            if ls.kind == "general_delta":
                p["rank"] = int(l["w_w2"].shape[1])
                p["b_a"], p["w0"] = f32(l["b_a"]), f32(l["w0"])
                self._matrix(p, "w_w2", mat(l["w_w2"]), None)
            else:
                a = ls.branches[0]
                p["bias"] = R.distance_bias_table(l["rel"].float().cpu(), a.bias_max, self.max_seq_len).to(dev).contiguous()
                for k in ("temp", "sink", "b_if", "out_l", "out_r"):
                    p[k] = f32(l[k])
                if p["fast"]:                        # (the MFMA kernels keep scores in the units of q . k)
                    p["bias"], p["sink"] = (p["bias"] / a.scale).contiguous(), (p["sink"] / a.scale).contiguous()
                self._matrix(p, "w_o_r", mat(l["w_o_r"]), None)
            if ls.has_ff:
                p.update({k: f32(l[k]) for k in ("ln2_w", "ln2_b", "b_rg2")})
                p["ln2_a"] = float(l["ln2_a"])
                if ls.moe is not None:
                    if ls.moe.experts > 256:
                        raise ValueError("up to 256 experts are supported")
                    self._matrix(p, "w_ff", torch.cat([mat(l["w_router"]), mat(l["w_rg2"])]), None)
                    p["w_gate_e"], p["w_up_e"], p["w_down_e"] = (mat(l[k]) for k in ("w_gate_e", "w_up_e", "w_down_e"))
                else:
                    self._matrix(p, "w_ff", torch.cat([mat(l["w_up"]), mat(l["w_rg2"])]), None)
                    self._matrix(p, "w_down", mat(l["w_down"]), None)
            self.layers.append(p)
            weights.layers[i] = {}
        if self._packed and spec.hidden_size % 128 == 0:
            self.lm_head_p = packing.pack_weight(self.lm_head)
            self._shapes.append((self.vocab_pad, spec.hidden_size, False))

    def _new_work_gated(self, rows: int):
        s, dev, at = self.spec, self.device, self.act_dtype
        z = lambda n, dt=torch.float32: torch.zeros(max(int(n), 1), device=dev, dtype=dt)
        B, H = min(rows, self.max_batch), s.hidden_size
        zc = wc = lc = oc = mc = m2 = z2 = ac = yc = qc = 1
        pairs = tiles = ef = 0
        for ls, p in zip(self.specs, self.layers):
            zc, yc = max(zc, self._cols(p, "w_in")), max(yc, self._cols(p, "w_o"))
            if p["fast"]:
                qc = max(qc, self._cols(p, "w_qkv"))
            if ls.kind == "general_delta":
                n = ls.heads * ls.dim
                wc, lc, oc, mc = max(wc, self._cols(p, "w_w2")), max(lc, p["rank"]), max(oc, n), max(mc, n)
            else:
                a, b = ls.branches
                mc, m2, oc = max(mc, a.heads * a.vdim), max(m2, b.heads * b.vdim), max(oc, b.heads * (b.vdim + 2))
                yc = max(yc, self._cols(p, "w_o_r"))
            if ls.has_ff:
                z2 = max(z2, self._cols(p, "w_ff"))
                if ls.moe is not None:
                    e = ls.moe
                    # (rows of the experts' sorted copies: whole tiles of 32 rows, or of 128 for steps with many rows)
                    pairs, ef = max(pairs, rows * e.top), max(ef, e.ff)
                    tiles = max(tiles, (rows * e.top + 31) // 32 + e.experts, 4 * ((rows * e.top + 127) // 128 + e.experts))
                else:
                    ac, yc = max(ac, ls.ff), max(yc, self._cols(p, "w_down"))
        ws_floats = self._ws_floats
        if self._packed and rows > self.decode_rows:
            for m_ in {rows, min(rows, 512), min(rows, 1024)}:
                if m_ > self.decode_rows:
                    ws_floats = max([ws_floats] + [int(self.K.gemm_ws_floats(m_, n_, k_)) for n_, k_, _ in self._shapes])
        i32 = torch.int32
        return SimpleNamespace(
            h=torch.zeros(rows, H, device=dev), xn=torch.zeros(rows, H, device=dev, dtype=at), z=z(rows * zc), wz=z(rows * wc),
            low=z(rows * lc, at), o=z(rows * oc), mixed=z(rows * mc, at), mixed2=z(rows * m2, at), ya=z(rows * yc), yb=z(rows * yc),
            z2=z(rows * z2), act=z(rows * ac, at), sel=z(pairs, i32), wts=z(pairs), pair_row=z(pairs, i32), tiles=z(1 + tiles, i32),
            row_tok=z(32 * tiles, i32), eact=z(32 * tiles * ef, at), ey=z(32 * tiles * H), ws=z(ws_floats + 4096),
            qkv16=z(rows * qc, torch.bfloat16),
            head_x=torch.zeros(B, H, device=dev, dtype=at), logits=torch.zeros(B, self.vocab_pad, device=dev), cmax=None, guided=False)

    def _layers_gated(self, wk, T: int, B: int, tok_pos, tok_seq, q_start, ctx, slots, max_q: int, lead_decode: int):
        K, eps, H = self.K, self.spec.norm_eps, self.spec.hidden_size
        h, xn = wk.h[:T], wk.xn[:T]
        view = lambda buf, cols: buf[:T * cols].view(T, cols)
        keep = self.keep_layer_outputs and not torch.cuda.is_current_stream_capturing()
        if keep:
            self.layer_outputs = []
        runs, first = self.runs, (self.spec.loop[0] if self.spec.loop else -1)

        def opening(ri):
            """(step vector, norm weight, bias, alpha) of what follows run ri - 1: the vector that opens a pass and the first norm of run ri."""
            if ri >= len(runs):
                return None, None, None, 0.0
            li, pas = runs[ri]
            p = self.layers[li]
            return (self.loop_step[pas] if pas >= 0 and li == first else None), p["ln1_w"], p["ln1_b"], p["ln1_a"]

        step, nw, nb, na = opening(0)
        K.dyt_gate(xn, h, None, None, None, None, None, None, step, nw, nb, None, na, eps)
        for ri, (li, _) in enumerate(runs):
            ls, p = self.specs[li], self.layers[li]
            z = view(wk.z, self._cols(p, "w_in"))
            self._mm(wk, z, xn, p, "w_in")
            ya, yb = view(wk.ya, self._cols(p, "w_o")), None
            if ls.kind == "general_delta":
                n, d, R = ls.heads * ls.dim, ls.dim, p["rank"]
                low, wz, o, mixed = view(wk.low, R), view(wk.wz, self._cols(p, "w_w2")), view(wk.o, n), view(wk.mixed, n)
                K.unary_act(low, z[:, 5 * n:5 * n + R], 1)
                self._mm(wk, wz, low, p, "w_w2")
                K.state_scan(0, o, z, wz[:, :n], self.rec[ri][0], None, p["b_a"], p["w0"], q_start, ctx, slots, ls.heads, d, d,
                             0, n, 2 * n, 4 * n, 0, 0, 1.0, 1.0, max_q, self.wmode == "bf16")
                K.headnorm_gate(mixed, o, z[:, 3 * n:4 * n], p["o_norm_w"], ls.heads, d, 0, eps)
                self._mm(wk, ya, mixed, p, "w_o")
                g0, wa, wb = 5 * n + R, None, None
            else:
                a, b = ls.branches
                qn, kn, vn, bn, bv = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim, b.heads * b.dim, b.heads * b.vdim
                c_g = 0 if p["fast"] else qn + kn + vn       # (z starts behind q | k | v when they have a GEMM of their own)
                c_q = c_g + a.heads
                c_k, c_v, c_rg, c_i = c_q + bn, c_q + 2 * bn, c_q + 2 * bn + bv, c_q + 2 * bn + 2 * bv
                mixed, mixed2, o = view(wk.mixed, a.heads * a.vdim), view(wk.mixed2, bv), view(wk.o, b.heads * (b.vdim + 2))
                gate = z[:, c_g:c_q]
                if p["fast"]:
                    Ha, G, d = a.heads, a.kv_heads, a.dim
                    qkv = view(wk.qkv16, self._cols(p, "w_qkv"))
                    self._mm(wk, qkv, xn, p, "w_qkv")
                    K.rope_kvwrite(qkv, None, 1, None, self.kv[ri], self._no_rope[d], self._no_rope[d], tok_pos, tok_seq,
                                   self.block_table, Ha, G, d, False)
                    ext = (p["temp"], p["bias"], p["sink"], gate)
                    if 0 < lead_decode < B and max_q > 1:
                        # single tokens riding in front of prompt portions: the decode-shaped kernel for them, the prefill-shaped for the rest
                        n = lead_decode
                        K.paged_attention_biased(mixed, qkv, self.kv[ri], q_start[:n + 1], ctx[:n], self.block_table, slots[:n], 1, Ha, G, d, a.scale, *ext)
                        K.paged_attention_biased(mixed, qkv, self.kv[ri], q_start[n:], ctx[n:], self.block_table, slots[n:], max_q, Ha, G, d, a.scale, *ext)
                    else:
                        K.paged_attention_biased(mixed, qkv, self.kv[ri], q_start, ctx, self.block_table, slots, max_q, Ha, G, d, a.scale, *ext)
                else:
                    kc, vc = self.kv[ri]
                    K.kv_store(z[:, :c_g], None, None, 0, kc, vc, tok_pos, tok_seq, self.block_table, a.kv_heads, a.dim, a.vdim, qn)
                    K.biased_attention(mixed, z, kc, vc, tok_pos, tok_seq, self.block_table, a.heads, a.kv_heads, a.dim, a.vdim, a.scale,
                                       p["temp"], p["bias"], p["sink"], gate)
                self._mm(wk, ya, mixed, p, "w_o")
                K.state_scan(1, o, z, None, self.rec[ri][0], self.rec[ri][1], p["b_if"], None, q_start, ctx, slots, b.heads, b.dim, b.vdim,
                             c_q, c_k, c_v, 0, c_i, c_i + b.heads, b.gate_cap, b.scale, max_q, self.wmode == "bf16")
                K.headnorm_gate(mixed2, o, z[:, c_rg:c_rg + bv], p["o_norm_w"], b.heads, b.vdim, 2, eps)
                yb = view(wk.yb, self._cols(p, "w_o"))
                self._mm(wk, yb, mixed2, p, "w_o_r")
                g0, wa, wb, yb = c_i + 2 * b.heads, p["out_l"], p["out_r"], yb[:, :H]
            if ls.has_ff:
                step, nw, nb, na = None, p["ln2_w"], p["ln2_b"], p["ln2_a"]
            else:
                step, nw, nb, na = opening(ri + 1)
            K.dyt_gate(xn if nw is not None else None, h, ya[:, :H], yb, wa, wb, z[:, g0:g0 + H], p["b_rg1"], step, nw, nb, None, na, eps)
            if ls.has_ff:
                z2 = view(wk.z2, self._cols(p, "w_ff"))
                self._mm(wk, z2, xn, p, "w_ff")
                if ls.moe is None:
                    act, ya = view(wk.act, ls.ff), view(wk.ya, self._cols(p, "w_down"))
                    K.unary_act(act, z2[:, :ls.ff], 0)
                    self._mm(wk, ya, act, p, "w_down")
                    g0 = ls.ff
                else:
                    e = ls.moe
                    # row tiles: 128 rows through the LDS-tiled kernel when the step has many rows (bf16, inner sizes in whole
                    # k-steps), else 32 rows through the register-tiled kernels; at most nt tiles hold a row
                    tr = 128 if (self.wmode == "bf16" and T * e.top >= 1024 and H % 32 == 0 and e.ff % 32 == 0) else 32
                    nt = (T * e.top + tr - 1) // tr + e.experts
                    eact, ey, ya = wk.eact[:tr * nt * e.ff].view(tr * nt, e.ff), wk.ey[:tr * nt * H].view(tr * nt, H), view(wk.ya, H)
                    K.moe_route(wk.sel, wk.wts, z2[:, :e.experts], e.top, e.groups, e.keep, e.scale)
                    K.moe_plan(wk.tiles, wk.row_tok, wk.pair_row, wk.sel, T * e.top, e.top, e.experts, tr)
                    K.moe_up(eact, xn, p["w_gate_e"], p["w_up_e"], wk.tiles, wk.row_tok, nt, e.limit, tr)
                    K.moe_down(ey, eact, p["w_down_e"], wk.tiles, wk.row_tok, nt, tr)
                    K.moe_combine(ya, ey, wk.pair_row, wk.wts, e.top)
                    g0 = e.experts
                step, nw, nb, na = opening(ri + 1)
                K.dyt_gate(xn if nw is not None else None, h, ya[:, :H], None, None, None, z2[:, g0:g0 + H], p["b_rg2"], step, nw, nb, None, na, eps)
            if keep:
                self.layer_outputs.append(h.clone())
        return None

    # ---- stacks with parallel layers on one norm -----------------------------------------------------------------------
    @staticmethod
    def _score_dim(ls) -> int:
        """Entries of one score map's keys."""
        return ls.kv_rank + ls.rot_dim if ls.kind == "latent_attention" else ls.dim

    def _par_rows(self, li: int) -> tuple:
        """(entries of a token's key row, of its value row) in the cache of attention layer li, over all its key / value heads.
        Latent attention keeps ONE row, the normed latent followed by the rotated key part; its values are the row's first
        entries (the matrix-core kernel wants them key-contiguous as well: a second, transposed copy of the latent)."""
        ls = self.specs[li]
        if ls.kind == "latent_attention":
            return ls.kv_rank + ls.rot_dim, ls.kv_rank if self._tile[li] else 0
        return ls.kv_heads * ls.maps * ls.dim, ls.kv_heads * ls.vdim

    def _load_par(self, weights: StageWeights, f32, mat):
        """Device weights of a stack with parallel layers. A mixer's input projections are ONE matrix; what a recurrence or a
        score needs in fp32 (gate matrices, decay rates, norm weights, rotation tables) stays fp32 in both modes."""
        from .rope import rope_table
        spec, dev = self.spec, self.device
        F = torch.nn.functional
        self.embed, self.lm_head, self.pos_embed = mat(weights.embed), mat(weights.lm_head), None
        self.lm_head_p = None
        self.final_norm_w = f32(weights.final_norm_w)
        self.vocab_pad = packing.padded_n(spec.vocab_size)
        self.layers = []
        tables: Dict[tuple, tuple] = {}
        for i, ls in enumerate(self.specs):
            l = weights.layers[i]
            p: Dict[str, object] = {k: f32(l[k]) for k in ("ln1_w", "ls1", "shift")}
            self._matrix(p, "w_in", mat(l["w_in"]), f32(l["b_in"]) if "b_in" in l else None)
            self._matrix(p, "w_o", mat(l["w_o"]), None)
            if ls.rope_dims:
                key = (ls.rope_dims, ls.rope_base, ls.rope_scaling)
                if key not in tables:
                    tables[key] = tuple(t.contiguous() for t in rope_table(ls.rope_dims, ls.rope_base, ls.rope_scaling, self.max_seq_len, dev))
                p["cos"], p["sin"] = tables[key]
            else:
                p["cos"] = p["sin"] = None
            if ls.kind == "rglru":
                p["conv_w"], p["conv_b"] = f32(l["conv_w"]), f32(l["conv_b"])
                # per block the decay gate's rows, then the input gate's: one block-diagonal product gives both
                p["w_g"] = torch.cat([f32(l["w_ra"]), f32(l["w_ri"])], dim=1).contiguous()
                p["b_g"] = torch.cat([f32(l["b_ra"]), f32(l["b_ri"])], dim=1).reshape(-1).contiguous()
                p["clam"] = (8.0 * F.softplus(f32(l["lam"]))).contiguous()
            elif ls.kind == "attention":
                lq1, lk1, lq2, lk2 = (f32(l[k]) for k in ("lq1", "lk1", "lq2", "lk2"))
                p["lam"] = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + ls.diff) if ls.maps == 2 else 0.0
            else:
                H, d, dr, dv, R = ls.heads, ls.dim, ls.rot_dim, ls.vdim, ls.kv_rank
                p["dq_norm"], p["dkv_norm"] = f32(l["dq_norm"]), f32(l["dkv_norm"])
                self._matrix(p, "w_uq", mat(l["w_uq"]), None)
                # per head: q . (W_uk c) = (W_uk^T q) . c, so the key up-projection moves to the query's side (the rotated
                # entries pass through an identity) and the cache keeps the latent alone
                wa = torch.zeros(H, R + dr, d + dr, device=dev, dtype=self.act_dtype)
                wa[:, :R, :d] = mat(l["w_uk"]).reshape(H, d, R).transpose(1, 2)
                wa[:, R:, d:] = torch.eye(dr, device=dev, dtype=self.act_dtype)
                p["w_abs"], p["w_uv"] = wa.contiguous(), mat(l["w_uv"]).reshape(H, dv, R).contiguous()
            if ls.ff:
                p["ls2"] = f32(l["ls2"])
                self._matrix(p, "w_up", mat(l["w_up"]), None)
                self._matrix(p, "w_down", mat(l["w_down"]), None)
                a = f32(l["act"]).reshape(-1)
                p["pq"] = torch.stack([F.softplus(a[0]), 0.5 + F.softplus(a[1])]).contiguous()
            self.layers.append(p)
            weights.layers[i] = {}
        if self._packed and spec.hidden_size % 128 == 0:
            self.lm_head_p = packing.pack_weight(self.lm_head)
            self._shapes.append((self.vocab_pad, spec.hidden_size, False))

    def _new_work_par(self, rows: int):
        s, dev, at = self.spec, self.device, self.act_dtype
        z = lambda n, dt=torch.float32: torch.zeros(max(int(n), 1), device=dev, dtype=dt)
        B, H = min(rows, self.max_batch), s.hidden_size
        zc = uc = mc = yc = z2 = ac = cq = q32 = q16 = qa = ol = 1
        for ls, p in zip(self.specs, self.layers):
            zc, yc = max(zc, self._cols(p, "w_in")), max(yc, self._cols(p, "w_o"))
            if ls.kind == "rglru":
                uc, mc = max(uc, ls.rec_width), max(mc, ls.rec_width)
            else:
                mc = max(mc, ls.heads * ls.vdim)
            if ls.kind == "latent_attention":
                cq, q32 = max(cq, ls.q_rank), max(q32, self._cols(p, "w_uq"))
                q16, qa = max(q16, ls.heads * (ls.dim + ls.rot_dim)), max(qa, ls.heads * (ls.kv_rank + ls.rot_dim))
                ol = max(ol, ls.heads * ls.kv_rank)
            if ls.kind == "attention":
                q16 = max(q16, ls.heads * ls.maps * ls.dim)
            if ls.ff:
                z2, ac, yc = max(z2, self._cols(p, "w_up")), max(ac, ls.ff), max(yc, self._cols(p, "w_down"))
        ws_floats = self._ws_floats
        if self._packed and rows > self.decode_rows:
            for m_ in {rows, min(rows, 512), min(rows, 1024)}:
                if m_ > self.decode_rows:
                    ws_floats = max([ws_floats] + [int(self.K.gemm_ws_floats(m_, n_, k_)) for n_, k_, _ in self._shapes])
        part = 1                  # partial results of the key splits of single-token steps (any number of rows up to B)
        for ls, tile in zip(self.specs, self._tile):
            if tile:
                dv = ls.kv_rank if ls.kind == "latent_attention" else ls.vdim
                part = max([part] + [int(self.K.tile_attention_part_floats(b_, ls.heads, ls.kv_heads, dv, ls.maps)) for b_ in range(1, B + 1)])
        scan = max([1] + [int(self.K.rglru_scan_ws_floats(rows, B, ls.rec_width)) for ls in self.specs if ls.kind == "rglru"])
        return SimpleNamespace(
            part=z(part), scan_ws=z(scan),
            h=torch.zeros(rows, H, device=dev), n32=torch.zeros(rows, H, device=dev), xn=torch.zeros(rows, H, device=dev, dtype=at),
            xs=torch.zeros(rows, H, device=dev, dtype=at), z=z(rows * zc), u=z(rows * uc), gates=z(rows * 2 * uc), mixed=z(rows * mc, at),
            ya=z(rows * yc), yb=z(rows * yc), z2=z(rows * z2), act=z(rows * ac, at), cq=z(rows * cq, at), q32=z(rows * q32),
            q16=z(rows * q16, at), qa=z(rows * qa), qa16=z(rows * qa if any(self._tile) else 1, at), olat=z(rows * ol, at), ws=z(ws_floats + 4096),
            head_x=torch.zeros(B, H, device=dev, dtype=at), logits=torch.zeros(B, self.vocab_pad, device=dev), cmax=None, guided=False)

    def _layers_par(self, wk, T: int, B: int, tok_pos, tok_seq, q_start, ctx, slots, max_q: int):
        K, eps, H = self.K, self.spec.norm_eps, self.spec.hidden_size
        h, n32, xn, xs = wk.h[:T], wk.n32[:T], wk.xn[:T], wk.xs[:T]
        view = lambda buf, cols: buf[:T * cols].view(T, cols)
        keep = self.keep_layer_outputs and not torch.cuda.is_current_stream_capturing()
        if keep:
            self.layer_outputs = []
        table, n_layers = self.block_table, len(self.layers)
        K.par_norm(xn, n32, h, None, None, None, None, self.layers[0]["ln1_w"], None, tok_seq, eps)
        for li, (ls, p) in enumerate(zip(self.specs, self.layers)):
            K.token_shift(xs, n32, self.rec[li][0], p["shift"], tok_pos, tok_seq)
            z = view(wk.z, self._cols(p, "w_in"))
            self._mm(wk, z, xs, p, "w_in")
            if ls.kind == "rglru":
                W, bw = ls.rec_width, ls.rec_width // ls.blocks
                u, gates, mixed = view(wk.u, W), view(wk.gates, 2 * W), view(wk.mixed, W)
                K.short_conv_act(u, z[:, W:2 * W], self.rec[li][1], p["conv_w"], p["conv_b"], q_start, ctx, slots, max_q, False)
                K.gemm_blocks(gates, u, p["w_g"], p["b_g"], bw, 2 * bw)
                K.rglru_scan(mixed, u, gates, z[:, :W], p["clam"], self.rec[li][2], q_start, ctx, slots, bw, max_q, wk.scan_ws)
            elif ls.kind == "attention":
                Hh, G, d, dv, M = ls.heads, ls.kv_heads, ls.dim, ls.vdim, ls.maps
                qn, kn, vn = Hh * M * d, G * M * d, G * dv
                kc, vc = self.kv[li]
                mixed = view(wk.mixed, Hh * dv)
                gate = z[:, qn + kn + vn:qn + kn + vn + Hh * dv] if ls.out_gate else None
                post = 1.0 - ls.diff if M == 2 else 1.0
                if self._tile[li]:
                    q16 = view(wk.q16, qn)
                    K.rope_cache_write(z, Hh * M, d, 0, q16, qn, z[:, qn:], kn, G * M, d, 0, kn, vn, True, kc, vc, ls.rope_dims,
                                       ls.rope_interleaved, p["cos"], p["sin"], tok_pos, tok_seq, table)
                    K.tile_attention(mixed, q16, M * d, kc, vc, q_start, ctx, slots, table, max_q, Hh, d, dv, M, ls.scale, ls.window or 0,
                                     ls.keep_first, ls.softcap, p["lam"], post, eps, gate, wk.part)
                else:
                    K.rope_cache_write(z, Hh * M, d, 0, None, 0, z[:, qn:], kn, G * M, d, 0, kn, vn, False, kc, vc, ls.rope_dims,
                                       ls.rope_interleaved, p["cos"], p["sin"], tok_pos, tok_seq, table)
                    K.multi_attention(mixed, z, M * d, kc, vc, 0, tok_pos, tok_seq, table, Hh, d, dv, M, ls.scale, ls.window or 0,
                                      ls.keep_first, ls.softcap, p["lam"], post, eps, gate)
            else:
                Hh, d, dr, dv, R, qr = ls.heads, ls.dim, ls.rot_dim, ls.vdim, ls.kv_rank, ls.q_rank
                kc, vc = self.kv[li]
                cq, q32 = view(wk.cq, qr), view(wk.q32, self._cols(p, "w_uq"))
                q16, qa, olat, mixed = view(wk.q16, Hh * (d + dr)), view(wk.qa, Hh * (R + dr)), view(wk.olat, Hh * R), view(wk.mixed, Hh * dv)
                K.norm32(cq, z[:, :qr], None, None, p["dq_norm"], None, eps, 0.0)
                K.norm32(z[:, qr:qr + R], z[:, qr:qr + R], None, None, p["dkv_norm"], None, eps, 0.0)       # (in place)
                self._mm(wk, q32, cq, p, "w_uq")
                tile = self._tile[li]
                K.rope_cache_write(q32, Hh, d + dr, d, q16, Hh * (d + dr), z[:, qr:], R + dr, 1, R + dr, R, 0, R if tile else 0, tile, kc,
                                   vc if tile else None, ls.rope_dims, ls.rope_interleaved, p["cos"], p["sin"], tok_pos, tok_seq, table)
                if tile:
                    qa16 = view(wk.qa16, Hh * (R + dr))
                    K.gemm_blocks(qa16, q16, p["w_abs"], None, d + dr, R + dr)
                    K.tile_attention(olat, qa16, R + dr, kc, vc, q_start, ctx, slots, table, max_q, Hh, R + dr, R, 1, ls.scale, 0, 0, 0.0,
                                     0.0, 1.0, eps, None, wk.part)
                else:
                    K.gemm_blocks(qa, q16, p["w_abs"], None, d + dr, R + dr)
                    K.multi_attention(olat, qa, R + dr, kc, kc, 0, tok_pos, tok_seq, table, Hh, R + dr, R, 1, ls.scale, 0, 0, 0.0, 0.0, 1.0,
                                      eps, None)
                K.gemm_blocks(mixed, olat, p["w_uv"], None, R, dv)
            ya, yb = view(wk.ya, self._cols(p, "w_o")), None
            self._mm(wk, ya, mixed, p, "w_o")
            if ls.ff:
                z2, act, yb = view(wk.z2, self._cols(p, "w_up")), view(wk.act, ls.ff), view(wk.yb, self._cols(p, "w_down"))
                self._mm(wk, z2, xn, p, "w_up")
                K.xielu(act, z2, p["pq"])
                self._mm(wk, yb, act, p, "w_down")
                yb = yb[:, :H]
            nxt = self.layers[li + 1]["ln1_w"] if li + 1 < n_layers else None
            K.par_norm(xn if nxt is not None else None, n32, h, ya[:, :H], yb, p["ls1"], p.get("ls2"), nxt, self.rec[li][0], tok_seq, eps)
            if keep:
                self.layer_outputs.append(h.clone())
        return None

    # ---- stacks with norms on the sublayers' outputs only --------------------------------------------------------------
    @staticmethod
    def _query_row(a) -> int:
        """Entries of one head's query as the attention kernel reads it: with mixed heads or head temperatures the mix is carried
        by the query, which then holds a part for every key head."""
        return a.kv_heads * a.dim if (a.head_mix or a.head_temp) else a.dim

    def _load_post(self, weights: StageWeights, f32, mat):
        """Device weights of a post-norm stack. Everything that reads the mixers' input is ONE matrix with the left branch's
        q | k | v biases in its epilogue; the router and the shared expert's gate | up are one more. What scores, norms and the
        recurrence need in fp32 (norm weights, the head mix, sinks, gate biases, rotation tables, routing corrections) stays
        fp32 in both modes."""
        from .rope import rope_table
        spec, dev = self.spec, self.device
        self.embed, self.pos_embed = mat(weights.embed), None
        self.lm_head, self.lm_head_p = self.embed, None
        self.final_norm_w = f32(weights.final_norm_w)
        self.vocab_pad = packing.padded_n(spec.vocab_size)
        self.layers = []
        tables: Dict[tuple, tuple] = {}
        for i, ls in enumerate(self.specs):
            l = weights.layers[i]
            a, b = ls.branches
            p: Dict[str, object] = {"ln1_w": f32(l["ln1_w"])}
            w_in = mat(l["w_in"])
            b_in = torch.zeros(w_in.shape[0], device=dev)
            if a.proj_bias:
                b_in[:l["b_qkv"].numel()] = f32(l["b_qkv"])
            self._matrix(p, "w_in", w_in, b_in)
            # a * (W_l m_l + b) + b' * W_r m_r = a * ([W_l | W_r] [m_l | (b' / a) m_r] + b): ONE output GEMM over both branches' mixed
            # rows, the ratio of the branch weights carried by the memory's norm weight (fp32), `a` applied where the sum is normed
            sa, sb = ls.branch_scales or (1.0, 1.0)
            w_l, b_l = mat(l["w_o"]), f32(l["b_o"]) if a.proj_bias else None
            if sa == 0.0:
                w_l, b_l, sa, sb = torch.zeros_like(w_l), None, 1.0, sb
            self._matrix(p, "w_o", torch.cat([w_l, mat(l["w_o_r"])], dim=1).contiguous(), b_l)
            p["out_scale"] = float(sa)
            p["q_norm_w"], p["k_norm_w"] = (f32(l["q_norm_w"]), f32(l["k_norm_w"])) if a.qk_norm else (None, None)
            # score_h = sum_g talk[h, g] temp[g] scale (q_g . k): the mix, the temperatures and the scale are one matrix
            p["mix"] = None
            if a.head_mix or a.head_temp:
                m = f32(l["talk"]) if a.head_mix else torch.eye(a.heads, device=dev)
                if a.head_temp:
                    m = m * f32(l["temp"]).view(1, -1)
                p["mix"] = (m * a.scale).contiguous()
            p["sink"] = (f32(l["sink"]) if a.sink_learned else torch.zeros(a.heads, device=dev)) if a.sink else None
            if a.rope_dims:
                key = (a.rope_dims, a.rope_base, a.rope_scaling)
                if key not in tables:
                    tables[key] = tuple(t.contiguous() for t in rope_table(a.rope_dims, a.rope_base, a.rope_scaling, self.max_seq_len, dev))
                p["cos"], p["sin"] = tables[key]
            else:
                p["cos"] = p["sin"] = None
            p["b_if"], p["o_norm_w"] = f32(l["b_if"]), (f32(l["o_norm_w"]) * (sb / sa)).contiguous()
            if ls.has_ff:
                p["ln2_w"] = f32(l["ln2_w"])
            if ls.moe is not None:
                e = ls.moe
                if e.outputs > 256:
                    raise ValueError("up to 256 router outputs are supported")
                ff_in = [mat(l["w_router"])] + ([mat(l["w_gate_s"]), mat(l["w_up_s"])] if e.shared_ff else [])
                self._matrix(p, "w_ff", torch.cat(ff_in), None)
                p["correction"] = f32(l["correction"]) if e.correction else None
                p["w_gate_e"], p["w_up_e"], p["w_down_e"] = (mat(l[k]) for k in ("w_gate_e", "w_up_e", "w_down_e"))
                if e.shared_ff:
                    self._matrix(p, "w_down_s", mat(l["w_down_s"]), None)
            elif ls.ff:
                self._matrix(p, "w_up", mat(l["w_up"]), f32(l["b_up"]))
                self._matrix(p, "w_down", mat(l["w_down"]), f32(l["b_down"]))
            self.layers.append(p)
            weights.layers[i] = {}
        if self._packed and spec.hidden_size % 128 == 0:
            self.lm_head_p = packing.pack_weight(self.lm_head)
            self._shapes.append((self.vocab_pad, spec.hidden_size, False))

    def _new_work_post(self, rows: int):
        s, dev, at = self.spec, self.device, self.act_dtype
        z = lambda n, dt=torch.float32: torch.zeros(max(int(n), 1), device=dev, dtype=dt)
        B, H = min(rows, self.max_batch), s.hidden_size
        zc = qc = oc = mc = m2 = yc = z2 = ac = sc = 1
        pairs = tiles = ef = 0
        part = 1                  # partial results of the key splits of single-token steps (any number of rows up to B)
        for ls, p, tile, direct in zip(self.specs, self.layers, self._tile, self._direct):
            a, b = ls.branches
            if direct:            # (and of the prompt steps' tiles)
                part = max(part, int(self.K.mixed_attention_part_floats(rows, a.heads, a.vdim)))
            zc, qc = max(zc, self._cols(p, "w_in")), max(qc, a.heads * self._query_row(a))
            mc, oc = max(mc, a.heads * a.vdim + b.heads * b.vdim), max(oc, b.heads * (b.vdim + 2))
            yc = max(yc, self._cols(p, "w_o"))
            if tile:
                gk = 1 if (a.head_mix or a.head_temp) else a.kv_heads      # (heads of the key cache)
                part = max([part] + [int(self.K.tile_attention_part_floats(b_, a.heads, a.kv_heads, a.vdim, 1, gk)) for b_ in range(1, B + 1)])
            if ls.moe is not None:
                e = ls.moe
                z2 = max(z2, self._cols(p, "w_ff"))
                # (rows of the experts' sorted copies: whole tiles of 32 rows, or of 128 for steps with many rows)
                pairs, ef = max(pairs, rows * e.top), max(ef, e.ff)
                tiles = max(tiles, (rows * e.top + 31) // 32 + e.experts, 4 * ((rows * e.top + 127) // 128 + e.experts))
                if e.shared_ff:
                    sc, yc = max(sc, e.shared_ff), max(yc, self._cols(p, "w_down_s"))
            elif ls.ff:
                z2, ac, yc = max(z2, self._cols(p, "w_up")), max(ac, ls.ff), max(yc, self._cols(p, "w_down"))
        ws_floats = self._ws_floats
        if self._packed and rows > self.decode_rows:
            for m_ in {rows, min(rows, 512), min(rows, 1024)}:
                if m_ > self.decode_rows:
                    ws_floats = max([ws_floats] + [int(self.K.gemm_ws_floats(m_, n_, k_)) for n_, k_, _ in self._shapes])
        i32 = torch.int32
        return SimpleNamespace(
            h=torch.zeros(rows, H, device=dev), xn=torch.zeros(rows, H, device=dev, dtype=at), z=z(rows * zc),
            qf=z(rows * qc, at if any(self._tile) else torch.float32), qf32=z(rows * qc if not all(self._tile) else 1),
            o=z(rows * oc), mixed=z(rows * mc, at), ya=z(rows * yc), yb=z(rows * yc), z2=z(rows * z2),
            act=z(rows * ac, at), acts=z(rows * sc, at), sel=z(pairs, i32), wts=z(pairs), pair_row=z(pairs, i32), tiles=z(1 + tiles, i32),
            row_tok=z(32 * tiles, i32), eact=z(32 * tiles * ef, at), ey=z(32 * tiles * H), part=z(part), ws=z(ws_floats + 4096),
            head_x=torch.zeros(B, H, device=dev, dtype=at), logits=torch.zeros(B, self.vocab_pad, device=dev), cmax=None, guided=False)

    def _layers_post(self, wk, T: int, B: int, tok_pos, tok_seq, q_start, ctx, slots, max_q: int):
        K, eps, H = self.K, self.spec.norm_eps, self.spec.hidden_size
        h, xn = wk.h[:T], wk.xn[:T]
        view = lambda buf, cols: buf[:T * cols].view(T, cols)
        keep = self.keep_layer_outputs and not torch.cuda.is_current_stream_capturing()
        if keep:
            self.layer_outputs = []
        table = self.block_table
        K.post_norm_add(xn, h, None, None, 1.0, 0.0, None, eps)         # the stream in the GEMMs' input type
        for li, (ls, p) in enumerate(zip(self.specs, self.layers)):
            a, b = ls.branches
            Hh, G, d, dv = a.heads, a.kv_heads, a.dim, a.vdim
            qn, kn, vn, gn, bn, bv = Hh * d, G * d, G * dv, (Hh * dv if a.out_gate else 0), b.heads * b.dim, b.heads * b.vdim
            # columns of the input projection: left q | k | v | g, right q | k | v | g | i | f
            c_g = qn + kn + vn
            c_q = c_g + Hh * dv
            c_k, c_v, c_rg, c_i, c_f = c_q + bn, c_q + 2 * bn, c_q + 2 * bn + bv, c_q + 2 * bn + 2 * bv, c_q + 2 * bn + 2 * bv + b.heads
            z = view(wk.z, self._cols(p, "w_in"))
            self._mm(wk, z, xn, p, "w_in")
            kc, vc = self.kv[li]
            tile, kd = self._tile[li], self._query_row(a)
            qf = view(wk.qf if tile else (wk.qf32 if wk.qf.dtype != torch.float32 else wk.qf), Hh * kd)
            both = view(wk.mixed, Hh * dv + bv)            # the two branches' mixed rows side by side: one output GEMM
            mixed, mixed2, o = both[:, :Hh * dv], both[:, Hh * dv:], view(wk.o, b.heads * (b.vdim + 2))
            gate = z[:, c_g:c_g + gn] if a.out_gate else None
            scale = 1.0 if p["mix"] is not None else a.scale
            if self._direct[li] and max_q > 1:
                # prompt portions (and whatever single tokens ride with them): plain queries, the mix on the score tiles
                q16 = view(wk.qf, Hh * d)
                K.mix_prep(z, Hh, G, d, dv, p["q_norm_w"], p["k_norm_w"], eps, a.rope_dims, p["cos"], p["sin"], a.v_norm, None, q16, kc, vc,
                           True, tok_pos, tok_seq, table)
                K.mixed_attention(mixed, q16, kc, vc, p["mix"], q_start, ctx, slots, table, max_q, Hh, d, dv, a.chunk, p["sink"], gate, wk.part)
                tile = None
            else:
                K.mix_prep(z, Hh, G, d, dv, p["q_norm_w"], p["k_norm_w"], eps, a.rope_dims, p["cos"], p["sin"], a.v_norm, p["mix"], qf, kc, vc,
                           tile, tok_pos, tok_seq, table)
            if tile is None:
                pass
            elif tile:
                K.tile_attention(mixed, qf, kd, kc, vc, q_start, ctx, slots, table, max_q, Hh, kd, dv, 1, scale, a.window or 0, 0, 0.0,
                                 0.0, 1.0, eps, gate, wk.part, a.chunk, p["sink"])
            else:
                K.multi_attention(mixed, qf, kd, kc, vc, 0, tok_pos, tok_seq, table, Hh, kd, dv, 1, scale, a.window or 0, 0, 0.0, 0.0,
                                  1.0, eps, gate, a.chunk, p["sink"])
            K.state_scan(1, o, z, None, self.rec[li][0], self.rec[li][1], p["b_if"], None, q_start, ctx, slots, b.heads, b.dim, b.vdim,
                         c_q, c_k, c_v, 0, c_i, c_f, b.gate_cap, b.scale, max_q, self.wmode == "bf16")
            K.headnorm_gate(mixed2, o, z[:, c_rg:c_rg + bv], p["o_norm_w"], b.heads, b.vdim, 2, eps)
            ya = view(wk.ya, self._cols(p, "w_o"))
            self._mm(wk, ya, both, p, "w_o")
            K.post_norm_add(xn, h, ya[:, :H], None, p["out_scale"], 0.0, p["ln1_w"], eps)
            if ls.moe is not None:
                e = ls.moe
                z2 = view(wk.z2, self._cols(p, "w_ff"))
                self._mm(wk, z2, xn, p, "w_ff")
                # row tiles: 128 rows through the LDS-tiled kernel when the step has many rows (bf16, inner sizes in whole
                # k-steps), else 32 rows through the register-tiled kernels; at most nt tiles hold a row
                tr = 128 if (self.wmode == "bf16" and T * e.top >= 1024 and H % 32 == 0 and e.ff % 32 == 0) else 32
                nt = (T * e.top + tr - 1) // tr + e.experts
                eact, ey, ya = wk.eact[:tr * nt * e.ff].view(tr * nt, e.ff), wk.ey[:tr * nt * H].view(tr * nt, H), view(wk.ya, H)
                K.moe_route(wk.sel, wk.wts, z2[:, :e.outputs], e.top, e.groups, e.keep, e.scale, p["correction"], e.score == "softmax",
                            e.group_rank, e.renorm)
                K.moe_plan(wk.tiles, wk.row_tok, wk.pair_row, wk.sel, T * e.top, e.top, e.experts, tr)
                K.moe_up(eact, xn, p["w_gate_e"], p["w_up_e"], wk.tiles, wk.row_tok, nt, e.limit if e.act != "silu" else 0.0, tr)
                K.moe_down(ey, eact, p["w_down_e"], wk.tiles, wk.row_tok, nt, tr)
                K.moe_combine(ya, ey, wk.pair_row, wk.wts, e.top, h if e.identity else None)
                yb = None
                if e.shared_ff:
                    acts, yb = view(wk.acts, e.shared_ff), view(wk.yb, self._cols(p, "w_down_s"))
                    K.unary_act(acts, z2[:, e.outputs:e.outputs + 2 * e.shared_ff], 3)
                    self._mm(wk, yb, acts, p, "w_down_s")
                    yb = yb[:, :H]
                K.post_norm_add(xn, h, ya, yb, 1.0, 1.0, p["ln2_w"], eps)
            elif ls.ff:
                z2, act, ya = view(wk.z2, self._cols(p, "w_up")), view(wk.act, ls.ff), view(wk.ya, self._cols(p, "w_down"))
                self._mm(wk, z2, xn, p, "w_up")
                K.unary_act(act, z2[:, :ls.ff], 2)
                self._mm(wk, ya, act, p, "w_down")
                K.post_norm_add(xn, h, ya[:, :H], None, 1.0, 0.0, p["ln2_w"], eps)
            if keep:
                self.layer_outputs.append(h.clone())
        return None

    def _fold(self, wk, T: int, pend):
        return None

    def _head(self, wk, rows_idx: torch.Tensor, R: int, T: int, pend):
        K = self.K
        hx = wk.head_x[:R]
        if self.gated:
            K.dyt_gate(hx, wk.h[:T], None, None, None, None, None, None, None, self.final_norm_w, self.final_norm_b, rows_idx[:R],
                       self.final_norm_a, self.spec.norm_eps)
        elif self.par or self.post:
            K.norm32(hx, wk.h[:T], None, None, self.final_norm_w, rows_idx[:R], self.spec.norm_eps, 0.0)
        else:
            K.norm32(hx, wk.h[:T], None, None, self.final_norm_w, rows_idx[:R], self.spec.norm_eps, 1.0)
        if self.lm_head_p is not None:
            K.gemm(wk.logits[:R], hx, self.lm_head_p, None, None, wk.ws, self.vocab_pad, 0, 0, 0)
        else:
            K.gemm_any(wk.logits[:R, :self.spec.vocab_size], hx, self.lm_head, None, 0)
        if self.spec.logit_softcap > 0:
            K.softcap(wk.logits[:R], self.spec.vocab_size, self.spec.logit_softcap)
        if self.spec.logit_scale != 1.0:
            K.scale_rows(wk.logits[:R], self.spec.vocab_size, self.spec.logit_scale)
        return wk.logits[:R]

    def memory_report(self) -> Dict[str, float]:
        gib = 1 << 30
        size = lambda t: t.numel() * t.element_size()
        wbytes = size(self.embed) + sum(size(t) for l in self.layers for t in l.values() if torch.is_tensor(t))
        kvb = sum(sum(size(t) for t in (kv if isinstance(kv, tuple) else (kv,))) for kv in (self.kv or []) if kv is not None)
        rec = sum(size(t) for r in self.rec if r is not None for t in r)
        return {"weights_gib": wbytes / gib, "kv_gib": kvb / gib, "state_gib": rec / gib, "kv_blocks": self.num_blocks,
                "kv_tokens": self.num_blocks * BLOCK}

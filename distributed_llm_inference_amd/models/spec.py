"""Architecture description of a decoder-only transformer.

A `ModelSpec` is everything the engine needs to know about a checkpoint's
architecture: it is parsed from a Hugging Face ``config.json`` (Llama family —
Llama, Mistral, Qwen2 — and GPT-2 family) or taken from the built-in table of
benchmark models.

The reference hard-codes one model name as a module constant and leans on
``AutoModelForCausalLM`` for everything else (orchestration.py:20,39-47;
Worker1.py:26,60-70).  Here the architecture is explicit so that each pipeline
stage can allocate exactly its own layers, KV cache and RoPE tables.
"""
from __future__ import annotations

import json
import os
import math
from dataclasses import dataclass, asdict, replace
from typing import Optional, Dict, Any


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` of a config.json. ``llama3``: Llama-3.1 frequency-dependent rescale (uses
    ``low_freq_factor`` / ``high_freq_factor``). ``linear``: positions divided by ``factor``. ``yarn``:
    interpolated below / extrapolated above a band of frequencies set by ``beta_fast`` / ``beta_slow``,
    cos and sin scaled by ``attention_factor`` (default 0.1 ln(factor) + 1). All of them are static, i.e. a
    table per stage; ``dynamic`` (a base that depends on the running sequence length) is refused."""
    factor: float = 8.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192
    rope_type: str = "llama3"
    beta_fast: float = 32.0
    beta_slow: float = 1.0
    attention_factor: Optional[float] = None
    truncate: bool = True
    # yarn: the ramp's width is max(high - low, 0.001) (a band that the clamps turn inside out counts as empty) instead of
    # high - low with only the equal case widened
    ramp_floor: bool = False


def distance_bucket(n: int, rows: int, far: int) -> int:
    """Row of a distance-bias table of `rows` rows for a distance n >= 0: one row per distance below rows / 2,
    then rows spaced logarithmically up to the distance `far`, the last row for everything beyond."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


@dataclass(frozen=True)
class LayerSpec:
    """One layer of a model whose layers differ from each other (a hybrid stack): which token mixer it
    has, the mixer's own sizes, and the width of its feed-forward sublayer (0: the layer has none).

    ``attention``: softmax attention over a paged cache, `heads` query heads over `kv_heads` key / value
    heads, queries and keys of `dim`, values of `vdim`; `window` (None: the whole context) keeps the
    keys j with 0 <= i - j < window; `sink` adds one to the softmax's denominator (a key of score 0 and no
    value); `scale` multiplies the scores; `rope` says whether positions rotate q and k; `v_mix`: the
    layer's values are blended with those of the first such layer of the stack, by a learned scalar.
    ``delta``: a gated delta-rule recurrence per head over a [dim, vdim] state, q / k shared by
    `heads // kv_heads` heads, each of q, k, v behind a causal convolution of `conv` taps.
    ``general_delta``: a delta rule with a decay per key channel (from a projection of low rank `rank`) and a
    removal rate per key channel along the unit key, over a [dim, dim] state per head.
    ``mlstm``: a matrix memory with exponential input / forget gates (log gates capped at `gate_cap`) kept in
    range by a running maximum, over a [dim, vdim] state, a [dim] normaliser and the maximum per head.
    ``parallel``: the mixers in `branches` read the same input; their outputs are RMS-normed over the width
    and averaged.
    ``rglru``: a real-gated linear recurrent unit over `rec_width` channels: one branch gelu_tanh(W_y h + b), the other
    W_x h + b behind a causal convolution of `conv` taps (with bias); per block of rec_width / `blocks` channels two
    gates sigmoid(square matrix . u + b); a = exp(-8 r softplus(lam)); S <- a S + sqrt(1 - a^2) i u; read-out S * y.
    ``latent_attention``: causal attention whose keys and values are expanded from a cached latent of `kv_rank` numbers
    per token (RMS-normed) plus one rotated key part of `rot_dim` shared by all heads; queries come through a latent of
    `q_rank` (RMS-normed) and carry `dim` unrotated + `rot_dim` rotated entries per head.
    Further switches of ``attention``: `bias_rows` > 0 adds a learned bias per (distance bucket, head) to the
    scaled scores (one bucket per distance below bias_rows / 2, logarithmic buckets up to `bias_max`);
    `head_temp` multiplies a head's scaled scores by a learned number; `sink_learned` makes the sink's score a
    learned number per head instead of 0; `head_gate` multiplies a head's output by the sigmoid of one more
    projection of the mixer's input. `maps` = 2: differential attention — q and k hold two maps per head, each a
    softmax attention of its own over the same values; the head's output is a1 - lambda a2 with
    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + `diff`, RMS-normed over the value size and scaled by 1 - `diff`.
    `keep_first`: with a window, the first keep_first tokens of the sequence stay visible. `softcap` > 0: scaled scores
    become cap tanh(score / cap). `out_gate`: the concatenated heads are multiplied by sigmoid(W_g h), element by element.
    `rope_dims` > 0: the first rope_dims entries of every q / k vector are rotated by position, frequencies
    `rope_base`^(-2i / rope_dims), pairs (2i, 2i + 1) when `rope_interleaved` else (i, i + rope_dims / 2), rescaled
    by `rope_scaling` when given.
    `proj_bias`: the q, k, v and output projections have biases. `qk_norm`: q and k are RMS-normed over the WHOLE projection
    (all heads at once, a learned weight per entry) before the rotation. `v_norm`: every head's value is divided by its root
    mean square (no weight) before it is cached. `head_mix`: the heads' scaled scores are mixed by a learned [heads, heads]
    matrix before mask and softmax, s_h <- sum_g M[h, g] s_g. `chunk` > 0: a query at i sees the keys j <= i of its own
    chunk only, floor(i / chunk) = floor(j / chunk), chunks counted from the sequence's position 0.
    ``parallel`` with `branch_scales` (a, b): the branches' outputs are added as a * left + b * right (no norms, no average).
    The feed-forward sublayer is `ff_kind`: ``gated_gelu`` (gelu_tanh(gate) * up, biases), ``gelu`` (up, exact
    GELU, down; no biases), ``xielu`` (up, a two-sided quadratic / exponential unit with two learned numbers, down),
    ``relu2`` (up, the square of relu, down; biases) or ``moe`` (`moe` says how tokens are routed to its experts)."""
    kind: str                       # "attention" | "delta" | "general_delta" | "mlstm" | "parallel" | "rglru" | "latent_attention"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    ff: int = 0
    window: Optional[int] = None
    scale: float = 1.0
    sink: bool = False
    rope: bool = False
    v_mix: bool = False
    conv: int = 0
    bias_rows: int = 0
    bias_max: int = 0
    head_temp: bool = False
    sink_learned: bool = False
    head_gate: bool = False
    gate_cap: float = 0.0
    rank: int = 0
    branches: tuple = ()
    ff_kind: str = "gated_gelu"
    moe: Optional["MoeSpec"] = None
    maps: int = 1
    diff: float = 0.0
    keep_first: int = 0
    softcap: float = 0.0
    out_gate: bool = False
    rope_dims: int = 0
    rope_base: float = 10000.0
    rope_interleaved: bool = False
    rope_scaling: Optional[RopeScaling] = None
    q_rank: int = 0
    kv_rank: int = 0
    rot_dim: int = 0
    rec_width: int = 0
    blocks: int = 1
    proj_bias: bool = False
    qk_norm: bool = False
    v_norm: bool = False
    head_mix: bool = False
    chunk: int = 0
    branch_scales: tuple = ()

    @property
    def group(self) -> int:
        return self.heads // self.kv_heads

    @property
    def has_state(self) -> bool:
        """The mixer keeps a per-sequence state in the sequence's slot."""
        return self.kind in ("delta", "general_delta", "mlstm", "rglru") or any(b.has_state for b in self.branches)

    @property
    def has_ff(self) -> bool:
        return self.ff > 0 or self.moe is not None

    @property
    def qk_heads(self) -> int:
        """Heads of the q projection: every query head for attention, the shared q / k heads for the delta rule."""
        return self.heads if self.kind == "attention" else self.kv_heads

    @property
    def v_heads(self) -> int:
        return self.kv_heads if self.kind == "attention" else self.heads

    def mixer_param_count(self, width: int) -> int:
        if self.kind == "rglru":
            w = self.rec_width
            return 3 * w * width + 2 * w * (w // self.blocks) + w * (self.conv + 6)
        if self.kind == "latent_attention":
            return width * (self.q_rank + self.kv_rank + self.rot_dim) + self.q_rank * self.heads * (self.dim + self.rot_dim) \
                + self.kv_rank * self.heads * (self.dim + self.vdim) + self.heads * self.vdim * width + self.q_rank + self.kv_rank
        if self.kind == "attention" and self.maps > 1:
            qn, kn = self.heads * self.maps * self.dim, self.kv_heads * self.maps * self.dim
            return width * (qn + kn + self.kv_heads * self.vdim + (2 if self.out_gate else 1) * self.heads * self.vdim) + 4 * self.dim
        if self.kind == "parallel":
            return sum(b.mixer_param_count(width) + width for b in self.branches)
        if self.kind == "general_delta":
            n = self.heads * self.dim
            return 6 * n * width + 2 * (self.rank or 16) * (width + n) // 2 + 3 * n
        if self.kind == "mlstm":
            return width * self.heads * (2 * self.dim + 3 * self.vdim + 2) + 2 * self.heads + self.heads * self.vdim
        qn, kn, vn = self.qk_heads * self.dim, self.kv_heads * self.dim, self.v_heads * self.vdim
        n = width * (qn + kn + vn) + self.heads * self.vdim * width
        if self.kind == "attention":
            return n + qn + kn + vn + 1
        return n + self.conv * (qn + kn + vn) + 2 * self.heads * width + 2 * self.heads + self.vdim + self.heads * self.vdim * width

    def ff_param_count(self, width: int) -> int:
        if self.moe is not None:
            return self.moe.experts * (3 * width * self.moe.ff + width) + 3 * width * self.moe.shared_ff
        if self.ff_kind in ("gelu", "xielu"):
            return 2 * width * self.ff
        if self.ff_kind == "relu2":
            return 2 * width * self.ff + self.ff + width
        return 3 * width * self.ff + 2 * self.ff + width if self.ff else 0


@dataclass(frozen=True)
class MoeSpec:
    """A routed feed-forward: `experts` small gated feed-forwards of width `ff`, of which a token runs `top`.
    Scores are the sigmoids of the router's logits. The experts are split into `groups` contiguous blocks of equal
    size; a block is ranked by its best two scores added up, and the choice is made among the experts of the
    `keep` best blocks. The outputs of the chosen experts are summed with weights score / (sum of the chosen
    scores) * `scale`. An
    expert computes down(g sigmoid(1.702 g) (u + 1)) with g = min(gate(x), limit), u = clamp(up(x), +-limit).
    Switches: `score` ``softmax``: scores are the softmax of the logits over all router outputs. `correction`: the CHOICE
    (of groups and of experts) goes by score + a learned number per router output, the weights by the score alone.
    `group_rank`: how many of a block's best choice scores are added up to rank it (1: its best). `renorm` off: the weights
    are the chosen scores times `scale`, not divided by their sum. `identity`: the router has that many outputs more than
    there are experts; choosing one of them returns the token's input itself (times the weight); they count as experts for
    the groups. `shared_ff` > 0: one more expert of that width runs for every token and is added unweighted. `act`
    ``silu``: an expert computes down(silu(gate(x)) * up(x)), no limits."""
    experts: int
    top: int
    ff: int
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    limit: float = 7.0
    score: str = "sigmoid"
    correction: bool = False
    group_rank: int = 2
    renorm: bool = True
    identity: int = 0
    shared_ff: int = 0
    act: str = "swish_lim"

    @property
    def outputs(self) -> int:
        """Outputs of the router: the experts and the identity experts."""
        return self.experts + self.identity


@dataclass(frozen=True)
class ModelSpec:
    name: str
    family: str                     # "llama" | "gpt2" | "letarax" | "nufapel" | "tezesun" | "zovozen"
    num_layers: int
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position: int
    norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: Optional[RopeScaling] = None
    tie_embeddings: bool = False
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None
    # further end-of-sequence ids (config.json / generation_config.json may list several: Llama-3-Instruct ends a
    # turn with <|eot_id|>, not with the id listed first)
    extra_eos_token_ids: tuple = ()
    # Llama-family variants: which config.json dialect the spec came from ("llama" | "mistral" | "qwen2"),
    # biases on the q/k/v projections (Qwen2; Llama with `attention_bias`) and on the output projection
    # (Llama with `attention_bias`), and the attention window of checkpoints trained with one (Mistral)
    hf_type: str = "llama"
    qkv_bias: bool = False
    o_bias: bool = False
    sliding_window: Optional[int] = None
    # hybrid stacks (family "letarax"): one entry per layer; the scalar fields above then hold the width, the
    # vocabulary and, for the sizes that differ per layer, the largest value over the layers
    layer_specs: tuple = ()
    # how a hybrid stack wraps its sublayers. "rms": RMS norms before and after every sublayer (weights stored as the
    # distance from one). "dyt": one dynamic-tanh norm tanh(alpha x) w + b before every sublayer (no statistics), also
    # as the final norm. `gated_residual`: a sublayer's output is multiplied by sigmoid(W h + b) of the sublayer's input
    norm_kind: str = "rms"
    gated_residual: bool = False
    # (start, stop, times): layers start .. stop-1 run `times` times in a row with the same weights, every pass with a
    # cache / state of its own and behind a learned vector added to the residual stream
    loop: tuple = ()
    learned_positions: bool = False          # a learned vector per position is added to the embedding
    logit_softcap: float = 0.0               # > 0: logits <- cap tanh(logits / cap)
    # `parallel_block`: a layer has ONE plain-weight RMS norm whose output both sublayers read: x += mixer(h) + ff(h).
    # `layer_scale`: each sublayer's output is multiplied by a learned vector before the sum. `token_shift`: what the
    # mixer reads is h + (previous token's h - h) * a learned vector (the previous h is per-sequence state of every layer)
    parallel_block: bool = False
    layer_scale: bool = False
    token_shift: bool = False
    logit_scale: float = 1.0                 # the logits are multiplied by it
    # `post_norm`: the sublayers read the residual stream itself and a plain-weight RMS norm sits on their OUTPUT only:
    # x += norm1(mixer(x)); x += norm2(ff(x))
    post_norm: bool = False

    @property
    def is_hybrid(self) -> bool:
        return bool(self.layer_specs)

    @property
    def has_recurrent_state(self) -> bool:
        """Some layer keeps a per-sequence state that lives in the sequence's slot (not in cache blocks): a sequence
        cannot change slots without its state being moved along."""
        return self.token_shift or any(l.has_state for l in self.layer_specs)

    def layer_runs(self):
        """[(layer, pass)] in the order the layers run; pass is -1 outside the repeated stretch, else the number of the
        pass (the stretch's first layer starts a pass). Every run owns a cache / state of its own."""
        n = len(self.layer_specs)
        if not self.loop:
            return [(i, -1) for i in range(n)]
        start, stop, times = self.loop
        runs = [(i, -1) for i in range(start)]
        for t in range(times):
            runs += [(i, t) for i in range(start, stop)]
        return runs + [(i, -1) for i in range(stop, n)]

    def check_context(self, max_seq_len: int):
        """Attention here is over the whole context. A checkpoint trained with a sliding window gives
        the same results only while no sequence is longer than the window."""
        if self.sliding_window is not None and max_seq_len > self.sliding_window:
            raise ValueError(f"{self.name}: sliding-window attention (window {self.sliding_window}) is not implemented; "
                             f"contexts up to the window are exact, max_seq_len={max_seq_len} is beyond it")

    # ---- derived quantities -------------------------------------------------
    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def qkv_size(self) -> int:
        return self.q_size + 2 * self.kv_size

    @property
    def group_size(self) -> int:
        return self.num_heads // self.num_kv_heads

    @property
    def is_llama(self) -> bool:
        return self.family == "llama"

    @property
    def is_gpt2(self) -> bool:
        return self.family == "gpt2"

    def layer_param_count(self) -> int:
        h, i = self.hidden_size, self.intermediate_size
        if self.is_hybrid:      # (the mean: the partitioner weighs layers equally)
            return sum(l.mixer_param_count(h) + l.ff_param_count(h) + (4 if l.ff else 2) * h for l in self.layer_specs) // len(self.layer_specs)
        if self.is_llama:
            return h * self.qkv_size + self.q_size * h + 3 * h * i + 2 * h + self._attn_bias_count()
        # GPT-2: c_attn, c_proj, c_fc, mlp c_proj, all with biases, two LayerNorms
        return (h * 3 * h + 3 * h) + (h * h + h) + (h * i + i) + (i * h + h) + 4 * h

    def attn_param_count(self) -> int:
        """Parameters of a layer's attention block (its norm, QKV and output projections)."""
        h = self.hidden_size
        if self.is_llama:
            return h * self.qkv_size + self.q_size * h + h + self._attn_bias_count()
        return (h * 3 * h + 3 * h) + (h * h + h) + 2 * h

    def _attn_bias_count(self) -> int:
        return (self.qkv_size if self.qkv_bias else 0) + (self.hidden_size if self.o_bias else 0)

    def embed_param_count(self) -> int:
        n = self.vocab_size * self.hidden_size
        if self.is_gpt2:
            n += self.max_position * self.hidden_size
        return n

    def head_param_count(self) -> int:
        """Final norm + lm_head (the lm_head matrix is read every step even when tied)."""
        return self.vocab_size * self.hidden_size + self.hidden_size * (2 if self.is_gpt2 else 1)

    def param_count(self) -> int:
        n = self.num_layers * self.layer_param_count() + self.embed_param_count()
        n += self.hidden_size * (2 if self.is_gpt2 else 1)
        if not self.tie_embeddings:
            n += self.vocab_size * self.hidden_size
        return n

    def kv_bytes_per_token_per_layer(self, dtype_bytes: int = 2) -> int:
        return 2 * self.num_kv_heads * self.head_dim * dtype_bytes

    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        return d

    @staticmethod
    def from_letarax_config(cfg: Dict[str, Any], name: str = "") -> "ModelSpec":
        """Letarax: a hybrid stack described layer by layer. ``layers`` lists for each layer its ``type``
        (``attention``: windowed softmax attention with a sink and no rotation, ``delta``: gated delta rule),
        the mixer's sizes (``mixer``: heads, kv_heads, dim, vdim; attention: mask.size, scale, v_mix;
        delta: conv) and its feed-forward (``mlp``: kind ``dense`` with ``ff``, or null). ``width``,
        ``vocab`` and ``norm.eps`` are the model's own. The output head is the embedding table."""
        layers = []
        for i, l in enumerate(cfg["layers"]):
            m, mlp = l["mixer"], l.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported (dense is)")
            ff = int(mlp["ff"]) if mlp is not None else 0
            if int(m["heads"]) % int(m["kv_heads"]):
                raise ValueError(f"layer {i}: {m['heads']} heads over {m['kv_heads']} key / value heads")
            common = dict(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), ff=ff)
            if l["type"] == "attention":
                win = (m.get("mask") or {}).get("size")
                layers.append(LayerSpec("attention", **common, window=int(win) if win else None,
                                        scale=float(m.get("scale", float(m["dim"]) ** -0.5)), sink=True, rope=False,
                                        v_mix=bool(m.get("v_mix", False))))
            elif l["type"] == "delta":
                layers.append(LayerSpec("delta", **common, conv=int(m["conv"]), scale=float(m["dim"]) ** -0.5))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        if not layers:
            raise ValueError("a model needs at least one layer")
        return ModelSpec(
            name=name or "letarax", family="letarax", num_layers=len(layers), hidden_size=int(cfg["width"]),
            num_heads=max(l.heads for l in layers), num_kv_heads=max(l.kv_heads for l in layers),
            head_dim=max(max(l.dim, l.vdim) for l in layers), intermediate_size=max(l.ff for l in layers),
            vocab_size=int(cfg["vocab"]), max_position=1 << 30, norm_eps=float(cfg["norm"]["eps"]),
            tie_embeddings=True, bos_token_id=cfg.get("bos_token_id"), eos_token_id=_scalar_eos(cfg.get("eos_token_id")),
            hf_type="letarax", layer_specs=tuple(layers))

    @staticmethod
    def from_nufapel_config(cfg: Dict[str, Any], name: str = "") -> "ModelSpec":
        """Nufapel: a hybrid stack listed layer by layer in ``layers``. A layer's ``type`` is ``general_delta`` (mixer:
        heads, dim) or ``parallel`` (mixer.left: attention with heads, kv_heads, dim, vdim, scale, bias_max, a distance-bias
        table, head temperatures, learned sinks and head gates; mixer.right: matrix memory with heads, dim, vdim,
        gate_cap); its ``mlp`` is null, ``dense`` (ff) or ``moe`` (expert.ff, expert.limit, router.experts / top / scale /
        groups.count / groups.keep). ``loop`` (start, stop, times) repeats a stretch of layers. Dynamic-tanh norms, gated
        residuals, learned positions (``max_positions``), a head of its own and ``logit_softcap``."""
        layers = []
        for i, l in enumerate(cfg["layers"]):
            m, mlp = l["mixer"], l.get("mlp")
            ffkw: Dict[str, Any] = dict(ff=0, ff_kind="gelu")
            if mlp is not None and mlp.get("kind", "dense") == "dense":
                ffkw = dict(ff=int(mlp["ff"]), ff_kind="gelu")
            elif mlp is not None and mlp["kind"] == "moe":
                r, e = mlp["router"], mlp["expert"]
                g = r.get("groups") or {}
                moe = MoeSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(e["ff"]), groups=int(g.get("count", 1)),
                              keep=int(g.get("keep", g.get("count", 1))), scale=float(r.get("scale", 1.0)), limit=float(e["limit"]))
                if moe.experts % moe.groups or not 1 <= moe.keep <= moe.groups or not 1 <= moe.top <= moe.keep * (moe.experts // moe.groups):
                    raise ValueError(f"layer {i}: {moe.experts} experts in {moe.groups} groups, {moe.keep} kept, {moe.top} chosen")
                ffkw = dict(ff=0, ff_kind="moe", moe=moe)
            elif mlp is not None:
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported (dense and moe are)")
            if l["type"] == "general_delta":
                layers.append(LayerSpec("general_delta", heads=int(m["heads"]), kv_heads=int(m["heads"]), dim=int(m["dim"]),
                                        vdim=int(m["dim"]), rank=int(m.get("rank", 0)), **ffkw))
            elif l["type"] == "parallel":
                a, b = m["left"], m["right"]
                if int(a["heads"]) % int(a["kv_heads"]):
                    raise ValueError(f"layer {i}: {a['heads']} heads over {a['kv_heads']} key / value heads")
                left = LayerSpec("attention", heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]), vdim=int(a["vdim"]),
                                 scale=float(a["scale"]), sink=True, sink_learned=True, head_temp=True, head_gate=True,
                                 bias_rows=int(a.get("bias_rows", 0)), bias_max=int(a["bias_max"]))
                right = LayerSpec("mlstm", heads=int(b["heads"]), kv_heads=int(b["heads"]), dim=int(b["dim"]), vdim=int(b["vdim"]),
                                  gate_cap=float(b["gate_cap"]), scale=float(b["dim"]) ** -0.5)
                layers.append(LayerSpec("parallel", heads=left.heads, kv_heads=left.kv_heads, dim=left.dim, vdim=left.vdim,
                                        branches=(left, right), **ffkw))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        if not layers:
            raise ValueError("a model needs at least one layer")
        loop = cfg.get("loop") or None
        lp = ()
        if loop and int(loop.get("times", 1)) >= 1 and int(loop["stop"]) > int(loop["start"]):
            lp = (int(loop["start"]), int(loop["stop"]), int(loop["times"]))
            if not 0 <= lp[0] < lp[1] <= len(layers):
                raise ValueError(f"loop {lp} does not fit {len(layers)} layers")
        heads = [b for l in layers for b in (l.branches or (l,))]
        return ModelSpec(
            name=name or "nufapel", family="nufapel", num_layers=len(layers), hidden_size=int(cfg["width"]),
            num_heads=max(l.heads for l in heads), num_kv_heads=max(l.kv_heads for l in heads),
            head_dim=max(max(l.dim, l.vdim) for l in heads),
            intermediate_size=max(max(l.ff, l.moe.ff if l.moe else 0) for l in layers),
            vocab_size=int(cfg["vocab"]), max_position=int(cfg["max_positions"]), norm_eps=float(cfg["norm"]["eps"]),
            tie_embeddings=False, bos_token_id=cfg.get("bos_token_id"), eos_token_id=_scalar_eos(cfg.get("eos_token_id")),
            hf_type="nufapel", layer_specs=tuple(layers), norm_kind="dyt", gated_residual=True, loop=lp,
            learned_positions=True, logit_softcap=float(cfg.get("logit_softcap") or 0.0))

    @staticmethod
    def from_tezesun_config(cfg: Dict[str, Any], name: str = "") -> "ModelSpec":
        """Tezesun: parallel layers (one RMS norm feeds the mixer and the feed-forward, both outputs scaled by learned
        vectors and added), the mixer's input blended with the previous token's. ``layers`` lists for each layer its
        ``type`` — ``rglru`` (mixer: width, blocks, conv), ``attention`` (differential: heads, kv_heads, dim, vdim, diff,
        scale, softcap, mask.size / mask.keep_first, rot.dims / base / scaling) or ``latent_attention`` (heads, dim,
        rot_dim, vdim, q_rank, kv_rank, scale, rot) — and its ``mlp`` (``dense`` with ``ff``, or null). A head of its own,
        logits times ``logit_scale``. Keys a config leaves out switch their mechanism off."""
        def rope_of(m, interleaved):
            rot = m.get("rot") or {}
            if not rot or not int(rot.get("dims", 0)):
                return dict(rope_dims=0)
            if int(rot["dims"]) % 2:
                raise ValueError("rot.dims must be even")
            sc, scaling = rot.get("scaling"), None
            if sc:
                scaling = RopeScaling(factor=float(sc["factor"]), rope_type="yarn", beta_fast=float(sc["fast"]), beta_slow=float(sc["slow"]),
                                      original_max_position_embeddings=int(sc["original"]), ramp_floor=True)
            return dict(rope_dims=int(rot["dims"]), rope_base=float(rot["base"]), rope_interleaved=interleaved, rope_scaling=scaling)

        layers = []
        for i, l in enumerate(cfg["layers"]):
            m, mlp = l["mixer"], l.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported (dense is)")
            ffkw = dict(ff=int(mlp["ff"]) if mlp is not None else 0, ff_kind="xielu")
            if l["type"] == "rglru":
                w, nb = int(m["width"]), int(m["blocks"])
                if w % nb:
                    raise ValueError(f"layer {i}: {w} channels in {nb} blocks")
                layers.append(LayerSpec("rglru", heads=nb, kv_heads=nb, dim=w // nb, vdim=w // nb, rec_width=w, blocks=nb,
                                        conv=int(m["conv"]), **ffkw))
            elif l["type"] == "attention":
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ValueError(f"layer {i}: {m['heads']} heads over {m['kv_heads']} key / value heads")
                mask = m.get("mask") or {}
                win = mask.get("size")
                layers.append(LayerSpec("attention", heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                                        window=int(win) if win else None, keep_first=int(mask.get("keep_first") or 0) if win else 0,
                                        scale=float(m["scale"]), softcap=float(m.get("softcap") or 0.0), maps=2, diff=float(m["diff"]),
                                        out_gate=True, **rope_of(m, True), **ffkw))
            elif l["type"] == "latent_attention":
                rp = rope_of(m, False)
                if rp["rope_dims"] > int(m["rot_dim"]):
                    raise ValueError(f"layer {i}: {rp['rope_dims']} rotated entries in a part of {m['rot_dim']}")
                layers.append(LayerSpec("latent_attention", heads=int(m["heads"]), kv_heads=1, dim=int(m["dim"]), vdim=int(m["vdim"]),
                                        scale=float(m["scale"]), q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]), rot_dim=int(m["rot_dim"]),
                                        **rp, **ffkw))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        if not layers:
            raise ValueError("a model needs at least one layer")
        att = [l for l in layers if l.kind != "rglru"] or layers
        return ModelSpec(
            name=name or "tezesun", family="tezesun", num_layers=len(layers), hidden_size=int(cfg["width"]),
            num_heads=max(l.heads for l in att), num_kv_heads=max(l.kv_heads for l in att),
            head_dim=max(max(l.dim, l.vdim) for l in att), intermediate_size=max(l.ff for l in layers),
            vocab_size=int(cfg["vocab"]), max_position=1 << 30, norm_eps=float(cfg["norm"]["eps"]), tie_embeddings=False,
            bos_token_id=cfg.get("bos_token_id"), eos_token_id=_scalar_eos(cfg.get("eos_token_id")), hf_type="tezesun",
            layer_specs=tuple(layers), parallel_block=True, layer_scale=True, token_shift=True,
            logit_scale=float(cfg.get("logit_scale", 1.0)))

    @staticmethod
    def from_zovozen_config(cfg: Dict[str, Any], name: str = "") -> "ModelSpec":
        """Zovozen: every layer is a ``parallel`` pair reading the residual stream itself, with RMS norms on the sublayers'
        outputs only. mixer.left: attention (heads, kv_heads, dim, vdim, scale, mask.size = chunk, rot.dims / base /
        scaling.factor) with biased projections, whole-projection q / k norms, unit values, head temperatures, mixed heads,
        learned sinks and an output gate; mixer.right: matrix memory (heads, dim, vdim, gate_cap); left_scale / right_scale
        weigh their sum. ``mlp``: null, ``dense`` (ff; squared relu, biases) or ``moe`` (expert.ff, router.experts / top /
        identity / groups.count / groups.keep, shared.ff). The head is the embedding table. Keys a config leaves out switch
        their mechanism off."""
        layers = []
        for i, l in enumerate(cfg["layers"]):
            m, mlp = l["mixer"], l.get("mlp")
            if l["type"] != "parallel":
                raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
            ffkw: Dict[str, Any] = dict(ff=0, ff_kind="relu2")
            if mlp is not None and mlp.get("kind", "dense") == "dense":
                ffkw = dict(ff=int(mlp["ff"]), ff_kind="relu2")
            elif mlp is not None and mlp["kind"] == "moe":
                r, g = mlp["router"], (mlp["router"].get("groups") or {})
                moe = MoeSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]), groups=int(g.get("count", 1)),
                              keep=int(g.get("keep", g.get("count", 1))), scale=1.0, limit=0.0, score="softmax", correction=True,
                              group_rank=1, renorm=False, identity=int(r.get("identity") or 0),
                              shared_ff=int((mlp.get("shared") or {}).get("ff") or 0), act="silu")
                if moe.outputs % moe.groups or not 1 <= moe.keep <= moe.groups or not 1 <= moe.top <= moe.keep * (moe.outputs // moe.groups):
                    raise ValueError(f"layer {i}: {moe.outputs} router outputs in {moe.groups} groups, {moe.keep} kept, {moe.top} chosen")
                ffkw = dict(ff=0, ff_kind="moe", moe=moe)
            elif mlp is not None:
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported (dense and moe are)")
            a, b = m["left"], m["right"]
            if int(a["heads"]) % int(a["kv_heads"]):
                raise ValueError(f"layer {i}: {a['heads']} heads over {a['kv_heads']} key / value heads")
            rot = a.get("rot") or {}
            rp: Dict[str, Any] = {}
            if int(rot.get("dims") or 0):
                if int(rot["dims"]) % 2 or int(rot["dims"]) > int(a["dim"]):
                    raise ValueError(f"layer {i}: {rot['dims']} rotated entries of {a['dim']}")
                f = float((rot.get("scaling") or {}).get("factor") or 1.0)
                rp = dict(rope_dims=int(rot["dims"]), rope_base=float(rot["base"]), rope_interleaved=False,
                          rope_scaling=RopeScaling(factor=f, rope_type="linear") if f != 1.0 else None)
            left = LayerSpec("attention", heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]), vdim=int(a["vdim"]),
                             scale=float(a["scale"]), sink=True, sink_learned=True, head_temp=True, out_gate=True, proj_bias=True,
                             qk_norm=True, v_norm=True, head_mix=True, chunk=int((a.get("mask") or {}).get("size") or 0), **rp)
            right = LayerSpec("mlstm", heads=int(b["heads"]), kv_heads=int(b["heads"]), dim=int(b["dim"]), vdim=int(b["vdim"]),
                              gate_cap=float(b["gate_cap"]), scale=float(b["dim"]) ** -0.5)
            layers.append(LayerSpec("parallel", heads=left.heads, kv_heads=left.kv_heads, dim=left.dim, vdim=left.vdim,
                                    branches=(left, right), branch_scales=(float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0))),
                                    **ffkw))
        if not layers:
            raise ValueError("a model needs at least one layer")
        heads = [b for l in layers for b in l.branches]
        return ModelSpec(
            name=name or "zovozen", family="zovozen", num_layers=len(layers), hidden_size=int(cfg["width"]),
            num_heads=max(l.heads for l in heads), num_kv_heads=max(l.kv_heads for l in heads),
            head_dim=max(max(l.dim, l.vdim) for l in heads),
            intermediate_size=max(max(l.ff, l.moe.ff if l.moe else 0, l.moe.shared_ff if l.moe else 0) for l in layers),
            vocab_size=int(cfg["vocab"]), max_position=1 << 30, norm_eps=float(cfg["norm"]["eps"]), tie_embeddings=True,
            bos_token_id=cfg.get("bos_token_id"), eos_token_id=_scalar_eos(cfg.get("eos_token_id")), hf_type="zovozen",
            layer_specs=tuple(layers), post_norm=True)

    def zovozen_config(self) -> Dict[str, Any]:
        """The inverse of `from_zovozen_config`."""
        out = []
        for l in self.layer_specs:
            a, b = l.branches
            left: Dict[str, Any] = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale}
            if a.chunk:
                left["mask"] = {"size": a.chunk}
            if a.rope_dims:
                left["rot"] = {"base": a.rope_base, "dims": a.rope_dims}
                if a.rope_scaling is not None:
                    left["rot"]["scaling"] = {"factor": a.rope_scaling.factor}
            m = {"left": left, "right": {"heads": b.heads, "dim": b.dim, "vdim": b.vdim, "gate_cap": b.gate_cap},
                 "left_scale": l.branch_scales[0], "right_scale": l.branch_scales[1]}
            if l.moe is not None:
                e = l.moe
                mlp: Optional[Dict[str, Any]] = {"kind": "moe", "expert": {"ff": e.ff},
                                                 "router": {"experts": e.experts, "top": e.top, "identity": e.identity,
                                                            "groups": {"count": e.groups, "keep": e.keep}}}
                if e.shared_ff:
                    mlp["shared"] = {"ff": e.shared_ff}
            else:
                mlp = {"kind": "dense", "ff": l.ff} if l.ff else None
            out.append({"type": "parallel", "mixer": m, "mlp": mlp})
        return {"architecture": "Zovozen", "layers": out, "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size,
                "width": self.hidden_size, "bos_token_id": self.bos_token_id, "eos_token_id": self.eos_token_id}

    def tezesun_config(self) -> Dict[str, Any]:
        """The inverse of `from_tezesun_config`."""
        def rot_of(l):
            if not l.rope_dims:
                return None
            r: Dict[str, Any] = {"base": l.rope_base, "dims": l.rope_dims}
            if l.rope_scaling is not None:
                rs = l.rope_scaling
                r["scaling"] = {"factor": rs.factor, "fast": rs.beta_fast, "slow": rs.beta_slow, "original": rs.original_max_position_embeddings}
            return r

        out = []
        for l in self.layer_specs:
            if l.kind == "rglru":
                m: Dict[str, Any] = {"width": l.rec_width, "blocks": l.blocks, "conv": l.conv}
            elif l.kind == "attention":
                m = {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale, "diff": l.diff}
                if l.softcap > 0:
                    m["softcap"] = l.softcap
                if l.window:
                    m["mask"] = {"size": l.window, "keep_first": l.keep_first}
            else:
                m = {"heads": l.heads, "dim": l.dim, "rot_dim": l.rot_dim, "vdim": l.vdim, "q_rank": l.q_rank, "kv_rank": l.kv_rank,
                     "scale": l.scale}
            if l.kind != "rglru" and rot_of(l) is not None:
                m["rot"] = rot_of(l)
            out.append({"type": l.kind, "mixer": m, "mlp": {"kind": "dense", "ff": l.ff} if l.ff else None})
        return {"architecture": "Tezesun", "layers": out, "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size,
                "width": self.hidden_size, "logit_scale": self.logit_scale, "bos_token_id": self.bos_token_id,
                "eos_token_id": self.eos_token_id}

    def nufapel_config(self) -> Dict[str, Any]:
        """The inverse of `from_nufapel_config` (`bias_rows` and `rank` are sizes a checkpoint's tensors give; they are
        written so that random weights of the same shapes can be drawn from the config alone)."""
        out = []
        for l in self.layer_specs:
            if l.kind == "general_delta":
                m: Dict[str, Any] = {"heads": l.heads, "dim": l.dim, "rank": l.rank}
            else:
                a, b = l.branches
                m = {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                              "bias_max": a.bias_max, "bias_rows": a.bias_rows},
                     "right": {"heads": b.heads, "dim": b.dim, "vdim": b.vdim, "gate_cap": b.gate_cap}}
            if l.moe is not None:
                e = l.moe
                mlp = {"kind": "moe", "expert": {"ff": e.ff, "limit": e.limit},
                       "router": {"experts": e.experts, "top": e.top, "scale": e.scale, "groups": {"count": e.groups, "keep": e.keep}}}
            else:
                mlp = {"kind": "dense", "ff": l.ff} if l.ff else None
            out.append({"type": l.kind, "mixer": m, "mlp": mlp})
        cfg = {"architecture": "Nufapel", "layers": out, "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size,
               "width": self.hidden_size, "max_positions": self.max_position, "logit_softcap": self.logit_softcap,
               "bos_token_id": self.bos_token_id, "eos_token_id": self.eos_token_id}
        if self.loop:
            cfg["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        return cfg

    def letarax_config(self) -> Dict[str, Any]:
        """The inverse of `from_letarax_config`."""
        out = []
        for l in self.layer_specs:
            if l.kind == "attention":
                m = {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale,
                     "mask": {"size": l.window}, "v_mix": l.v_mix}
            else:
                m = {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "conv": l.conv}
            out.append({"type": l.kind, "mixer": m, "mlp": {"kind": "dense", "ff": l.ff} if l.ff else None})
        return {"architecture": "Letarax", "layers": out, "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size,
                "width": self.hidden_size, "bos_token_id": self.bos_token_id, "eos_token_id": self.eos_token_id}

    # ---- constructors ------------------------------------------------------
    @staticmethod
    def from_hf_config(cfg: Dict[str, Any], name: str = "") -> "ModelSpec":
        """Build a spec from the dict form of a Hugging Face ``config.json``."""
        mt = cfg.get("model_type", "")
        archs = cfg.get("architectures") or []
        if cfg.get("architecture") == "Letarax":
            return ModelSpec.from_letarax_config(cfg, name=name)
        if cfg.get("architecture") == "Nufapel":
            return ModelSpec.from_nufapel_config(cfg, name=name)
        if cfg.get("architecture") == "Tezesun":
            return ModelSpec.from_tezesun_config(cfg, name=name)
        if cfg.get("architecture") == "Zovozen":
            return ModelSpec.from_zovozen_config(cfg, name=name)
        if mt == "gpt2" or any("GPT2" in a for a in archs):
            if cfg.get("activation_function", "gelu_new") != "gelu_new" or cfg.get("scale_attn_by_inverse_layer_idx"):
                raise ValueError("GPT-2 variants other than gelu_new MLPs with plain 1/sqrt(d) attention scaling are not supported")
            h = cfg.get("n_embd", cfg.get("hidden_size"))
            nh = cfg.get("n_head", cfg.get("num_attention_heads"))
            inner = cfg.get("n_inner") or 4 * h
            return ModelSpec(
                name=name or cfg.get("_name_or_path", "gpt2"),
                family="gpt2",
                num_layers=cfg.get("n_layer", cfg.get("num_hidden_layers")),
                hidden_size=h,
                num_heads=nh,
                num_kv_heads=nh,
                head_dim=h // nh,
                intermediate_size=inner,
                vocab_size=cfg["vocab_size"],
                max_position=cfg.get("n_positions", cfg.get("max_position_embeddings", 1024)),
                norm_eps=cfg.get("layer_norm_epsilon", 1e-5),
                tie_embeddings=True,
                bos_token_id=cfg.get("bos_token_id"),
                eos_token_id=_scalar_eos(cfg.get("eos_token_id")),
            )
        # (a config.json without model_type that has the Llama keys is taken as Llama; a NAMED other architecture is
        # refused rather than run as if it were one: Gemma, Phi, ... differ in norms, activations and scalings)
        if mt in ("llama", "mistral", "qwen2") or any(a.startswith(("Llama", "Mistral", "Qwen2For")) for a in archs) \
                or (not mt and not archs and "num_key_value_heads" in cfg):
            if cfg.get("hidden_act", "silu") not in ("silu", "swish"):
                raise ValueError(f"hidden_act {cfg.get('hidden_act')!r} is not supported (the fused MLP epilogue is SiLU-gated)")
            if float(cfg.get("partial_rotary_factor", 1.0)) != 1.0:
                raise ValueError("partial rotary embeddings are not supported")
            h = cfg["hidden_size"]
            nh = cfg["num_attention_heads"]
            rs = cfg.get("rope_scaling")
            rope_theta = cfg.get("rope_theta")
            # transformers >= 5 nests theta/scaling under `rope_parameters`
            rp = cfg.get("rope_parameters")
            if isinstance(rp, dict):
                rope_theta = rp.get("rope_theta", rope_theta)
                if rp.get("rope_type", "default") not in ("default", None):
                    rs = rp
            scaling = None
            rtype = rs.get("rope_type", rs.get("type")) if isinstance(rs, dict) else None
            if rtype == "llama3":
                scaling = RopeScaling(
                    factor=float(rs.get("factor", 8.0)),
                    low_freq_factor=float(rs.get("low_freq_factor", 1.0)),
                    high_freq_factor=float(rs.get("high_freq_factor", 4.0)),
                    original_max_position_embeddings=int(rs.get("original_max_position_embeddings", 8192)),
                )
            elif rtype == "linear":
                scaling = RopeScaling(factor=float(rs["factor"]), rope_type="linear",
                                      original_max_position_embeddings=int(cfg.get("max_position_embeddings", 2048)))
            elif rtype == "yarn":
                if rs.get("mscale") or rs.get("mscale_all_dim"):
                    raise ValueError("yarn rope_scaling with mscale / mscale_all_dim is not supported")
                orig = int(rs.get("original_max_position_embeddings") or cfg.get("max_position_embeddings", 2048))
                factor = rs.get("factor")
                scaling = RopeScaling(
                    factor=float(factor if factor is not None else cfg.get("max_position_embeddings", orig) / orig),
                    rope_type="yarn", original_max_position_embeddings=orig,
                    beta_fast=float(rs.get("beta_fast") or 32.0), beta_slow=float(rs.get("beta_slow") or 1.0),
                    attention_factor=(float(rs["attention_factor"]) if rs.get("attention_factor") is not None else None),
                    truncate=bool(rs.get("truncate", True)))
            elif rtype not in (None, "default"):
                raise ValueError(f"rope_scaling type {rtype!r} is not supported (llama3, linear and yarn are)")
            if cfg.get("mlp_bias"):
                raise ValueError("mlp_bias=true is not supported (the fused gate/up epilogue has no bias)")
            hf_type = mt if mt in ("mistral", "qwen2") else "llama"
            attn_bias = bool(cfg.get("attention_bias", False))
            window = cfg.get("sliding_window")
            if hf_type == "qwen2" and not cfg.get("use_sliding_window", False):
                window = None
            if hf_type == "llama":
                window = None
            return ModelSpec(
                name=name or cfg.get("_name_or_path", "llama"),
                family="llama",
                num_layers=cfg["num_hidden_layers"],
                hidden_size=h,
                num_heads=nh,
                num_kv_heads=cfg.get("num_key_value_heads", nh),
                head_dim=cfg.get("head_dim") or h // nh,
                intermediate_size=cfg["intermediate_size"],
                vocab_size=cfg["vocab_size"],
                max_position=cfg.get("max_position_embeddings", 2048),
                norm_eps=cfg.get("rms_norm_eps", 1e-5),
                rope_theta=float(rope_theta if rope_theta is not None else 10000.0),
                rope_scaling=scaling,
                tie_embeddings=bool(cfg.get("tie_word_embeddings", False)),
                bos_token_id=cfg.get("bos_token_id"),
                eos_token_id=_scalar_eos(cfg.get("eos_token_id")),
                extra_eos_token_ids=_more_eos(cfg.get("eos_token_id")),
                hf_type=hf_type,
                qkv_bias=True if hf_type == "qwen2" else attn_bias,       # Qwen2: q/k/v always biased, o never
                o_bias=False if hf_type == "qwen2" else attn_bias,
                sliding_window=int(window) if window else None,
            )
        raise ValueError(f"unsupported model_type {mt!r} (architectures={archs})")

    @staticmethod
    def from_pretrained(path_or_name: str) -> "ModelSpec":
        """Resolve a built-in model name or a local directory holding ``config.json``."""
        key = path_or_name.lower()
        if key in BUILTIN_SPECS:
            return BUILTIN_SPECS[key]
        short = key.split("/")[-1]
        if short in BUILTIN_SPECS and not os.path.isdir(path_or_name):
            return BUILTIN_SPECS[short]
        cfg_path = os.path.join(path_or_name, "config.json")
        if os.path.isfile(cfg_path):
            with open(cfg_path) as f:
                spec = ModelSpec.from_hf_config(json.load(f), name=path_or_name)
            # generation_config.json may name more end-of-sequence ids than config.json does
            gen_path = os.path.join(path_or_name, "generation_config.json")
            if os.path.isfile(gen_path):
                with open(gen_path) as f:
                    ge = json.load(f).get("eos_token_id")
                ids = [int(x) for x in (ge if isinstance(ge, (list, tuple)) else [ge] if ge is not None else [])]
                more = tuple(dict.fromkeys(x for x in (*spec.extra_eos_token_ids, *ids) if x != spec.eos_token_id))
                if spec.eos_token_id is None and more:
                    spec = replace(spec, eos_token_id=more[0], extra_eos_token_ids=more[1:])
                else:
                    spec = replace(spec, extra_eos_token_ids=more)
            return spec
        raise FileNotFoundError(
            f"{path_or_name!r} is neither a built-in model ({sorted(BUILTIN_SPECS)}) "
            f"nor a directory with config.json (the Hugging Face hub is not reachable)")

    def hf_config(self) -> Dict[str, Any]:
        """The inverse of `from_hf_config`: a config.json dict for this spec."""
        if self.is_hybrid:
            return {"nufapel": self.nufapel_config, "tezesun": self.tezesun_config, "zovozen": self.zovozen_config}.get(self.family, self.letarax_config)()
        if self.is_gpt2:
            return {
                "model_type": "gpt2", "architectures": ["GPT2LMHeadModel"],
                "n_layer": self.num_layers, "n_embd": self.hidden_size, "n_head": self.num_heads,
                "n_inner": self.intermediate_size, "vocab_size": self.vocab_size,
                "n_positions": self.max_position, "layer_norm_epsilon": self.norm_eps,
                "activation_function": "gelu_new",
                "bos_token_id": self.bos_token_id, "eos_token_id": self.eos_token_id,
            }
        cfg = {
            "model_type": "llama", "architectures": ["LlamaForCausalLM"],
            "num_hidden_layers": self.num_layers, "hidden_size": self.hidden_size,
            "num_attention_heads": self.num_heads, "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim, "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size, "max_position_embeddings": self.max_position,
            "rms_norm_eps": self.norm_eps, "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_embeddings, "hidden_act": "silu",
            "attention_bias": self.qkv_bias, "mlp_bias": False,
            "bos_token_id": self.bos_token_id, "eos_token_id": self.eos_token_id,
        }
        if self.hf_type == "qwen2":
            cfg.update({"model_type": "qwen2", "architectures": ["Qwen2ForCausalLM"],
                        "use_sliding_window": self.sliding_window is not None, "sliding_window": self.sliding_window,
                        "max_window_layers": 0})
            del cfg["attention_bias"], cfg["mlp_bias"], cfg["head_dim"]
        elif self.hf_type == "mistral":
            cfg.update({"model_type": "mistral", "architectures": ["MistralForCausalLM"],
                        "sliding_window": self.sliding_window})
            del cfg["attention_bias"], cfg["mlp_bias"]
        elif self.qkv_bias != self.o_bias:
            raise ValueError("a Llama config.json has one `attention_bias` for q/k/v and o alike")
        if self.extra_eos_token_ids:
            cfg["eos_token_id"] = [self.eos_token_id, *self.extra_eos_token_ids]
        if self.rope_scaling is not None:
            rs = self.rope_scaling
            if rs.rope_type == "linear":
                cfg["rope_scaling"] = {"rope_type": "linear", "factor": rs.factor}
            elif rs.rope_type == "yarn":
                cfg["rope_scaling"] = {"rope_type": "yarn", "factor": rs.factor, "beta_fast": rs.beta_fast, "beta_slow": rs.beta_slow,
                                       "original_max_position_embeddings": rs.original_max_position_embeddings,
                                       "truncate": rs.truncate}
                if rs.attention_factor is not None:
                    cfg["rope_scaling"]["attention_factor"] = rs.attention_factor
            else:
                cfg["rope_scaling"] = {
                    "rope_type": "llama3", "factor": rs.factor, "low_freq_factor": rs.low_freq_factor,
                    "high_freq_factor": rs.high_freq_factor,
                    "original_max_position_embeddings": rs.original_max_position_embeddings,
                }
        return cfg


def _scalar_eos(v):
    if isinstance(v, (list, tuple)):
        return v[0] if v else None
    return v


def _more_eos(v) -> tuple:
    return tuple(int(x) for x in v[1:]) if isinstance(v, (list, tuple)) else ()


# Shapes of the benchmark models.  The reference serves TinyLlama-1.1B-Chat
# (orchestration.py:20); GPT-2 small and Llama-3 8B/70B are the other benchmark shapes.
BUILTIN_SPECS: Dict[str, ModelSpec] = {
    "gpt2": ModelSpec(
        name="gpt2", family="gpt2", num_layers=12, hidden_size=768, num_heads=12, num_kv_heads=12,
        head_dim=64, intermediate_size=3072, vocab_size=50257, max_position=1024, norm_eps=1e-5,
        tie_embeddings=True, bos_token_id=50256, eos_token_id=50256),
    "tinyllama-1.1b": ModelSpec(
        name="TinyLlama/TinyLlama-1.1B-Chat-v1.0", family="llama", num_layers=22, hidden_size=2048,
        num_heads=32, num_kv_heads=4, head_dim=64, intermediate_size=5632, vocab_size=32000,
        max_position=2048, norm_eps=1e-5, rope_theta=10000.0, bos_token_id=1, eos_token_id=2),
    "llama-3-8b": ModelSpec(
        name="meta-llama/Meta-Llama-3-8B", family="llama", num_layers=32, hidden_size=4096,
        num_heads=32, num_kv_heads=8, head_dim=128, intermediate_size=14336, vocab_size=128256,
        max_position=8192, norm_eps=1e-5, rope_theta=500000.0, bos_token_id=128000, eos_token_id=128001),
    "llama-3-70b": ModelSpec(
        name="meta-llama/Meta-Llama-3-70B", family="llama", num_layers=80, hidden_size=8192,
        num_heads=64, num_kv_heads=8, head_dim=128, intermediate_size=28672, vocab_size=128256,
        max_position=8192, norm_eps=1e-5, rope_theta=500000.0, bos_token_id=128000, eos_token_id=128001),
    # Llama-family variants: Mistral (trained with a 4096-token attention window: exact up to there) and
    # Qwen2 (biases on the q/k/v projections, tied embeddings at this size)
    "mistral-7b": ModelSpec(
        name="mistralai/Mistral-7B-v0.1", family="llama", num_layers=32, hidden_size=4096, num_heads=32,
        num_kv_heads=8, head_dim=128, intermediate_size=14336, vocab_size=32000, max_position=32768,
        norm_eps=1e-5, rope_theta=10000.0, bos_token_id=1, eos_token_id=2, hf_type="mistral", sliding_window=4096),
    "qwen2.5-3b": ModelSpec(
        name="Qwen/Qwen2.5-3B", family="llama", num_layers=36, hidden_size=2048, num_heads=16, num_kv_heads=2,
        head_dim=128, intermediate_size=11008, vocab_size=151936, max_position=32768, norm_eps=1e-6,
        rope_theta=1000000.0, tie_embeddings=True, bos_token_id=151643, eos_token_id=151643,
        hf_type="qwen2", qkv_bias=True),
    # GQA groups that are not powers of two: 3 query heads per kv head (Llama-3.2-3B), 7 (Qwen2.5-7B)
    "llama-3.2-3b": ModelSpec(
        name="meta-llama/Llama-3.2-3B", family="llama", num_layers=28, hidden_size=3072, num_heads=24, num_kv_heads=8,
        head_dim=128, intermediate_size=8192, vocab_size=128256, max_position=131072, norm_eps=1e-5,
        rope_theta=500000.0, rope_scaling=RopeScaling(32.0, 1.0, 4.0, 8192), tie_embeddings=True,
        bos_token_id=128000, eos_token_id=128001),
    "qwen2.5-7b": ModelSpec(
        name="Qwen/Qwen2.5-7B", family="llama", num_layers=28, hidden_size=3584, num_heads=28, num_kv_heads=4,
        head_dim=128, intermediate_size=18944, vocab_size=152064, max_position=131072, norm_eps=1e-6,
        rope_theta=1000000.0, bos_token_id=151643, eos_token_id=151643, hf_type="qwen2", qkv_bias=True),
}
# aliases
BUILTIN_SPECS["mistral-7b-v0.1"] = BUILTIN_SPECS["mistral-7b"]
BUILTIN_SPECS["tinyllama"] = BUILTIN_SPECS["tinyllama-1.1b"]
BUILTIN_SPECS["tinyllama-1.1b-chat-v1.0"] = BUILTIN_SPECS["tinyllama-1.1b"]
BUILTIN_SPECS["gpt2-small"] = BUILTIN_SPECS["gpt2"]
BUILTIN_SPECS["llama3-8b"] = BUILTIN_SPECS["llama-3-8b"]
BUILTIN_SPECS["meta-llama-3-8b"] = BUILTIN_SPECS["llama-3-8b"]
BUILTIN_SPECS["llama3-70b"] = BUILTIN_SPECS["llama-3-70b"]
BUILTIN_SPECS["meta-llama-3-70b"] = BUILTIN_SPECS["llama-3-70b"]


def letarax_spec(name: str, width: int, heads: int, kv_heads: int, head_dim: int, ff: int, num_layers: int, window: int,
                 vocab_size: int = 32000, conv: int = 4, pattern: str = "adaa") -> ModelSpec:
    """A Letarax stack from a few numbers: `pattern` repeats over the layers ('a' windowed attention with the sink and
    value mixing, 'd' gated delta rule), every layer with a feed-forward of `ff`, keys and values of `head_dim`."""
    att = LayerSpec("attention", heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=head_dim, ff=ff, window=window,
                    scale=head_dim ** -0.5, sink=True, v_mix=True)
    dlt = LayerSpec("delta", heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=head_dim, ff=ff, conv=conv, scale=head_dim ** -0.5)
    layers = tuple(att if pattern[i % len(pattern)] == "a" else dlt for i in range(num_layers))
    return ModelSpec(name=name, family="letarax", num_layers=num_layers, hidden_size=width, num_heads=heads, num_kv_heads=kv_heads,
                     head_dim=head_dim, intermediate_size=ff, vocab_size=vocab_size, max_position=1 << 30, norm_eps=1e-5,
                     tie_embeddings=True, bos_token_id=1, eos_token_id=2, hf_type="letarax", layer_specs=layers)


def nufapel_spec(name: str, width: int, heads: int, kv_heads: int, head_dim: int, ff: int, num_layers: int, vocab_size: int = 32000,
                 pattern: str = "pgpp", experts: int = 8, top: int = 2, loop: tuple = (), max_position: int = 8192, rank: int = 64,
                 bias_rows: int = 32, bias_max: int = 2048) -> ModelSpec:
    """A Nufapel stack from a few numbers: `pattern` repeats over the layers ('p': attention with distance bias, head temperature,
    learned sink and head gate beside a matrix memory of half as many heads; 'g': generalised delta rule over width / head_dim
    heads); 'g' layers have a dense feed-forward of `ff`, 'p' layers a routed one of `experts` experts of ff / 4, `top` chosen."""
    moe = MoeSpec(experts=experts, top=top, ff=max(8, ff // 4), groups=max(1, experts // 4), keep=max(1, experts // 8), scale=1.0, limit=7.0)
    left = LayerSpec("attention", heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=head_dim, scale=head_dim ** -0.5, sink=True,
                     sink_learned=True, head_temp=True, head_gate=True, bias_rows=bias_rows, bias_max=bias_max)
    right = LayerSpec("mlstm", heads=max(1, heads // 2), kv_heads=max(1, heads // 2), dim=head_dim, vdim=head_dim, gate_cap=15.0, scale=head_dim ** -0.5)
    par = LayerSpec("parallel", heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=head_dim, branches=(left, right), ff=0, ff_kind="moe", moe=moe)
    gh = max(1, width // head_dim)
    gd = LayerSpec("general_delta", heads=gh, kv_heads=gh, dim=head_dim, vdim=head_dim, rank=rank, ff=ff, ff_kind="gelu")
    layers = tuple(par if pattern[i % len(pattern)] == "p" else gd for i in range(num_layers))
    return ModelSpec(name=name, family="nufapel", num_layers=num_layers, hidden_size=width, num_heads=heads, num_kv_heads=kv_heads,
                     head_dim=head_dim, intermediate_size=ff, vocab_size=vocab_size, max_position=max_position, norm_eps=1e-5,
                     tie_embeddings=False, bos_token_id=1, eos_token_id=2, hf_type="nufapel", layer_specs=layers, norm_kind="dyt",
                     gated_residual=True, loop=loop, learned_positions=True, logit_softcap=30.0)


def tezesun_spec(name: str, width: int, heads: int, kv_heads: int, head_dim: int, ff: int, num_layers: int, window: int = 1024,
                 vocab_size: int = 32000, pattern: str = "lrra", blocks: int = 0, conv: int = 4, q_rank: int = 0, kv_rank: int = 0,
                 rot_dim: int = 0, keep_first: int = 4) -> ModelSpec:
    """A Tezesun stack from a few numbers: `pattern` repeats over the layers ('r' recurrent unit over `width` channels, 'a'
    differential attention whose two maps have head_dim / 2 entries each and whose values have head_dim, window + kept
    first tokens, rescaled interleaved rotation, 'l' latent attention with head_dim unrotated entries per head), every
    layer with a feed-forward of `ff`."""
    rot_dim = rot_dim or max(2, head_dim // 2)
    rec = LayerSpec("rglru", heads=blocks or heads, kv_heads=blocks or heads, dim=width // (blocks or heads), vdim=width // (blocks or heads),
                    rec_width=width, blocks=blocks or heads, conv=conv, ff=ff, ff_kind="xielu")
    dm = max(2, head_dim // 2)
    att = LayerSpec("attention", heads=heads, kv_heads=kv_heads, dim=dm, vdim=head_dim, window=window, keep_first=keep_first,
                    scale=dm ** -0.5, softcap=30.0, maps=2, diff=0.5, out_gate=True, rope_dims=dm, rope_base=1000000.0, rope_interleaved=True,
                    rope_scaling=RopeScaling(factor=4.0, rope_type="yarn", beta_fast=32.0, beta_slow=1.0, original_max_position_embeddings=4096,
                                             ramp_floor=True),
                    ff=ff, ff_kind="xielu")
    lat = LayerSpec("latent_attention", heads=heads, kv_heads=1, dim=head_dim, vdim=head_dim, scale=(head_dim + rot_dim) ** -0.5,
                    q_rank=q_rank or max(8, width // 2), kv_rank=kv_rank or max(8, width // 8), rot_dim=rot_dim, rope_dims=rot_dim,
                    rope_base=10000.0, ff=ff, ff_kind="xielu")
    kinds = {"r": rec, "a": att, "l": lat}
    layers = tuple(kinds[pattern[i % len(pattern)]] for i in range(num_layers))
    return ModelSpec(name=name, family="tezesun", num_layers=num_layers, hidden_size=width, num_heads=heads, num_kv_heads=kv_heads,
                     head_dim=head_dim, intermediate_size=ff, vocab_size=vocab_size, max_position=1 << 30, norm_eps=1e-5,
                     tie_embeddings=False, bos_token_id=1, eos_token_id=2, hf_type="tezesun", layer_specs=layers, parallel_block=True,
                     layer_scale=True, token_shift=True, logit_scale=1.5)


def zovozen_spec(name: str, width: int, heads: int, kv_heads: int, head_dim: int, ff: int, num_layers: int, vocab_size: int = 32000,
                 pattern: str = "md", experts: int = 8, top: int = 2, identity: int = 2, groups: int = 5, keep: int = 2, chunk: int = 1024,
                 vdim: int = 0, rot_dims: int = 0, mem_heads: int = 0, shared: bool = True) -> ModelSpec:
    """A Zovozen stack from a few numbers: every layer is attention (biased projections, whole-projection q / k norms, unit
    values, half-rotated heads with linearly rescaled frequencies, head temperatures, mixed heads, learned sinks, chunked
    mask, output gate) beside a matrix memory of `mem_heads` heads (half as many by default); `pattern` repeats over the
    layers' feed-forwards: 'd' dense squared-relu of `ff`, 'm' routed (`experts` experts of ff / 4 plus `identity` identity
    experts in `groups` groups, `top` chosen from `keep` groups, a shared expert of ff / 2), 'n' none."""
    moe = MoeSpec(experts=experts, top=top, ff=max(8, ff // 4), groups=groups, keep=keep, scale=1.0, limit=0.0, score="softmax",
                  correction=True, group_rank=1, renorm=False, identity=identity, shared_ff=max(8, ff // 2) if shared else 0, act="silu")
    rd = rot_dims or max(2, head_dim // 2)
    left = LayerSpec("attention", heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=vdim or head_dim, scale=head_dim ** -0.5, sink=True,
                     sink_learned=True, head_temp=True, out_gate=True, proj_bias=True, qk_norm=True, v_norm=True, head_mix=True, chunk=chunk,
                     rope_dims=rd, rope_base=500000.0, rope_scaling=RopeScaling(factor=4.0, rope_type="linear"))
    mh = mem_heads or max(1, heads // 2)
    right = LayerSpec("mlstm", heads=mh, kv_heads=mh, dim=head_dim, vdim=vdim or head_dim, gate_cap=12.0, scale=head_dim ** -0.5)
    par = dict(heads=heads, kv_heads=kv_heads, dim=head_dim, vdim=vdim or head_dim, branches=(left, right), branch_scales=(0.75, 0.6))
    kinds = {"d": LayerSpec("parallel", ff=ff, ff_kind="relu2", **par), "m": LayerSpec("parallel", ff=0, ff_kind="moe", moe=moe, **par),
             "n": LayerSpec("parallel", ff=0, ff_kind="relu2", **par)}
    layers = tuple(kinds[pattern[i % len(pattern)]] for i in range(num_layers))
    return ModelSpec(name=name, family="zovozen", num_layers=num_layers, hidden_size=width, num_heads=heads, num_kv_heads=kv_heads,
                     head_dim=max(head_dim, vdim), intermediate_size=ff, vocab_size=vocab_size, max_position=1 << 30, norm_eps=1e-5,
                     tie_embeddings=True, bos_token_id=1, eos_token_id=2, hf_type="zovozen", layer_specs=layers, post_norm=True)


# Letarax stacks of the sizes of the Llama benchmark shapes (random weights; `bench.py --hybrid-compare` runs them)
BUILTIN_SPECS["letarax-1b-like"] = letarax_spec("letarax-1b-like", 2048, 16, 4, 128, 8192, 8, 1024)
BUILTIN_SPECS["letarax-8b-like"] = letarax_spec("letarax-8b-like", 4096, 32, 8, 128, 14336, 4, 2048)
# Nufapel stacks of the same sizes (`bench.py --gated-compare` runs them beside the Letarax stacks)
BUILTIN_SPECS["nufapel-1b-like"] = nufapel_spec("nufapel-1b-like", 2048, 16, 4, 128, 8192, 8)
BUILTIN_SPECS["nufapel-8b-like"] = nufapel_spec("nufapel-8b-like", 4096, 32, 8, 128, 14336, 4)
# Tezesun stacks of the same sizes (`bench.py --parallel-compare` runs them beside the Letarax stacks)
BUILTIN_SPECS["tezesun-1b-like"] = tezesun_spec("tezesun-1b-like", 2048, 16, 4, 128, 8192, 8, window=1024, kv_rank=448, rot_dim=64, q_rank=1024)
BUILTIN_SPECS["tezesun-8b-like"] = tezesun_spec("tezesun-8b-like", 4096, 32, 8, 128, 14336, 4, window=2048, kv_rank=448, rot_dim=64, q_rank=1536)
# Zovozen stacks of the same sizes (`bench.py --postnorm-compare` runs them beside the Nufapel stacks)
BUILTIN_SPECS["zovozen-1b-like"] = zovozen_spec("zovozen-1b-like", 2048, 16, 4, 128, 8192, 8, chunk=1024)
BUILTIN_SPECS["zovozen-8b-like"] = zovozen_spec("zovozen-8b-like", 4096, 32, 8, 128, 14336, 4, chunk=2048)


def _register_test_models():
    # resolvable by name in spawned stage processes too (tests of the multi-process pipeline)
    BUILTIN_SPECS["tiny-llama-test"] = tiny_spec("llama")
    BUILTIN_SPECS["tiny-gpt2-test"] = tiny_spec("gpt2")
    BUILTIN_SPECS["tiny-llama-8l-test"] = tiny_spec("llama", name="tiny-llama-8l-test", num_layers=8)   # splits into 8 stages
    BUILTIN_SPECS["tiny-llama-gpu-test"] = tiny_spec(
        "llama", name="tiny-llama-gpu-test", hidden_size=256, num_heads=4, num_kv_heads=2, head_dim=64,
        intermediate_size=512, vocab_size=320, num_layers=4)
    BUILTIN_SPECS["tiny-qwen2-gpu-test"] = tiny_spec(
        "llama", name="tiny-qwen2-gpu-test", hidden_size=256, num_heads=4, num_kv_heads=2, head_dim=64,
        intermediate_size=512, vocab_size=320, num_layers=4, hf_type="qwen2", qkv_bias=True, tie_embeddings=True)
    BUILTIN_SPECS["tiny-letarax-test"] = letarax_spec("tiny-letarax-test", 64, 4, 2, 16, 96, 4, 12, vocab_size=320, conv=3, pattern="ada")
    BUILTIN_SPECS["tiny-letarax-gpu-test"] = letarax_spec("tiny-letarax-gpu-test", 128, 4, 2, 64, 256, 4, 40, vocab_size=320)
    BUILTIN_SPECS["tiny-nufapel-test"] = nufapel_spec("tiny-nufapel-test", 64, 4, 2, 16, 96, 3, vocab_size=320, pattern="pgp", experts=4,
                                                      loop=(0, 2, 2), max_position=256, rank=8, bias_rows=8, bias_max=64)
    BUILTIN_SPECS["tiny-nufapel-gpu-test"] = nufapel_spec("tiny-nufapel-gpu-test", 128, 4, 2, 32, 256, 4, vocab_size=320, experts=8,
                                                          loop=(1, 3, 2), max_position=512, rank=16, bias_rows=16, bias_max=200)
    BUILTIN_SPECS["tiny-tezesun-test"] = tezesun_spec("tiny-tezesun-test", 64, 4, 2, 16, 96, 4, window=12, vocab_size=320, conv=3, blocks=4,
                                                      q_rank=24, kv_rank=20, rot_dim=8, keep_first=3)
    BUILTIN_SPECS["tiny-tezesun-gpu-test"] = tezesun_spec("tiny-tezesun-gpu-test", 128, 4, 2, 32, 256, 4, window=36, vocab_size=320, blocks=2,
                                                          q_rank=48, kv_rank=40, rot_dim=16, keep_first=5)
    BUILTIN_SPECS["tiny-zovozen-test"] = zovozen_spec("tiny-zovozen-test", 64, 4, 2, 16, 96, 3, vocab_size=320, pattern="dmn", experts=6,
                                                      identity=2, groups=4, keep=2, chunk=20, vdim=24, rot_dims=8)
    BUILTIN_SPECS["tiny-zovozen-gpu-test"] = zovozen_spec("tiny-zovozen-gpu-test", 128, 4, 2, 32, 256, 4, vocab_size=320, pattern="mdm",
                                                          experts=6, identity=2, groups=2, keep=1, chunk=40, vdim=48, rot_dims=16)
    BUILTIN_SPECS["tiny-gpt2-gpu-test"] = tiny_spec(
        "gpt2", name="tiny-gpt2-gpu-test", hidden_size=256, num_heads=4, num_kv_heads=4, head_dim=64,
        intermediate_size=1024, vocab_size=333, num_layers=4)


def tiny_spec(family: str = "llama", **overrides) -> ModelSpec:
    """A toy architecture for unit tests (seconds on CPU)."""
    if family == "llama":
        base = dict(name="tiny-llama-test", family="llama", num_layers=4, hidden_size=128, num_heads=4,
                    num_kv_heads=2, head_dim=32, intermediate_size=256, vocab_size=320, max_position=256,
                    norm_eps=1e-5, rope_theta=10000.0, bos_token_id=1, eos_token_id=2)
    else:
        base = dict(name="tiny-gpt2-test", family="gpt2", num_layers=4, hidden_size=128, num_heads=4,
                    num_kv_heads=4, head_dim=32, intermediate_size=512, vocab_size=320, max_position=256,
                    norm_eps=1e-5, tie_embeddings=True, bos_token_id=0, eos_token_id=0)
    base.update(overrides)
    return ModelSpec(**base)


_register_test_models()

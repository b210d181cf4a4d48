"""Prefill and decode throughput of a Letarax stack beside a Llama stack of equal size (`bench.py --hybrid-compare`), of a
Nufapel stack beside the Letarax stack of equal size (`bench.py --gated-compare`), of a Tezesun stack beside the
Letarax stack of equal size (`bench.py --parallel-compare`), and of a Zovozen stack beside the Nufapel stack of equal size
(`bench.py --postnorm-compare`).

Both models get random weights and the same width, head counts, head size, feed-forward width, depth and
vocabulary; the Letarax stack has three attention layers (windowed, with the sink and value mixing) to one delta-rule
layer. Each is built by the launcher's `build_executor` and driven through the executor's own step
functions: `forward` on one ragged prefill step, `decode_step` on a fixed-shape micro-batch (hipGraph replays).
Times are HIP events around the timed steps; one JSON line per size goes to stdout.
"""
from __future__ import annotations

import json
import sys
import time

SIZES = {
    # name: width, heads, kv heads, head size, feed-forward, layers, window
    "1b-like": (2048, 16, 4, 128, 8192, 8, 1024),
    "8b-like": (4096, 32, 8, 128, 14336, 4, 2048),
}
VOCAB = 32000


def gated_specs(name: str):
    """The Nufapel stack of a size beside the closest existing design of the same size: the Letarax stack (both keep an fp32
    residual stream, attention over the paged cache beside recurrent layers with slot-resident state)."""
    from distributed_llm_inference_amd.models.spec import BUILTIN_SPECS
    return BUILTIN_SPECS[f"nufapel-{name}"], BUILTIN_SPECS[f"letarax-{name}"]


def parallel_specs(name: str):
    """The Tezesun stack of a size (latent attention, two recurrent units, differential attention, repeated) beside the closest
    existing design of the same width, heads, feed-forward and depth: the Letarax stack (fp32 residual stream, windowed
    attention over the paged cache beside recurrent layers with slot-resident state)."""
    from distributed_llm_inference_amd.models.spec import BUILTIN_SPECS
    return BUILTIN_SPECS[f"tezesun-{name}"], BUILTIN_SPECS[f"letarax-{name}"]


def postnorm_specs(name: str):
    """The Zovozen stack of a size (attention with mixed heads, chunked mask and sink beside a matrix memory; routed and dense
    feed-forwards alternating) beside the closest existing design of the same width, heads, head size, feed-forward and
    depth: the Nufapel stack (attention beside a matrix memory in three layers of four, routed feed-forwards)."""
    from distributed_llm_inference_amd.models.spec import BUILTIN_SPECS
    return BUILTIN_SPECS[f"zovozen-{name}"], BUILTIN_SPECS[f"nufapel-{name}"]


def specs(name: str):
    from distributed_llm_inference_amd.models.spec import BUILTIN_SPECS, ModelSpec
    W, H, G, D, F, L, win = SIZES[name]
    hyb = BUILTIN_SPECS[f"letarax-{name}"]
    assert (hyb.hidden_size, hyb.num_heads, hyb.num_kv_heads, hyb.head_dim, hyb.intermediate_size, hyb.num_layers) == (W, H, G, D, F, L)
    llama = ModelSpec(name=f"llama-{name}", family="llama", num_layers=L, hidden_size=W, num_heads=H, num_kv_heads=G,
                      head_dim=D, intermediate_size=F, vocab_size=VOCAB, max_position=8192, norm_eps=1e-5, tie_embeddings=True)
    return hyb, llama


def build(spec, rows: int, chunk: int, seq: int):
    from distributed_llm_inference_amd.config import EngineConfig
    from distributed_llm_inference_amd.models.partition import make_plans
    from distributed_llm_inference_amd.parallel.launcher import build_executor
    blocks = rows * ((seq + 31) // 32) + 8
    cfg = EngineConfig(model=spec.name, weights="random", dtype="bf16", pp_size=1, max_batch=rows, num_micro_batches=1,
                       max_seq_len=seq, prefill_chunk=chunk, kv_blocks=blocks, device="cuda", backend="hip", seed=1)
    return build_executor(cfg, spec, make_plans(spec, 1)[0])


def _step(slots, q, ctx, toks=None, tables=None, replay=False):
    from distributed_llm_inference_amd.runtime.batch import StepBatch
    B = len(slots)
    return StepBatch(slots=list(slots), q_lens=[q] * B, ctx_lens=[ctx] * B, sample=[1] * B, temperature=[0.0] * B, top_k=[1] * B,
                     top_p=[1.0] * B, seeds=[0] * B, sample_steps=[0] * B, token_ids=toks, replay=replay,
                     table_slots=list(slots) if tables else [], table_blocks=tables or [])


def time_prefill(ex, seqs: int, length: int, iters: int) -> float:
    """Seconds per prefill step of `seqs` prompts of `length` tokens (ragged step, contexts start empty)."""
    import torch
    per = (length + 31) // 32
    tables = [list(range(i * per, (i + 1) * per)) for i in range(seqs)]
    toks = torch.randint(0, VOCAB, (seqs * length,), dtype=torch.int32)
    ex.forward(_step(range(seqs), length, 0, toks.tolist(), tables), toks)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        ex.forward(_step(range(seqs), length, 0, toks.tolist()), toks)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / 1e3 / iters


def time_decode(ex, rows: int, ctx: int, iters: int) -> float:
    """Seconds per decode step of `rows` sequences that hold `ctx` tokens (captured step, replayed)."""
    import torch
    per = (ctx + iters + 40) // 32 + 1
    tables = [list(range(i * per, (i + 1) * per)) for i in range(rows)]
    d = _step(range(rows), 1, ctx, [1] * rows, tables)
    ex.decode_step(d)
    for _ in range(3):
        ex.decode_step(_step(range(rows), 1, 0, None, None, replay=True))
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        ex.decode_step(_step(range(rows), 1, 0, None, None, replay=True))
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / 1e3 / iters


def main(sizes=None, iters: int = 8, out=sys.stdout, gated: bool = False, parallel: bool = False, postnorm: bool = False) -> int:
    import gc
    import torch
    rows, ctx, plen = 64, 1024, 2048
    for name in (sizes or list(SIZES)):
        rec = {"metric": "zovozen_vs_nufapel_tokens_per_s" if postnorm else "tezesun_vs_letarax_tokens_per_s" if parallel else "nufapel_vs_letarax_tokens_per_s" if gated else "letarax_vs_llama_tokens_per_s", "size": name, "dtype": "bf16", "data": "synthetic", "weights": "random",
               "config": dict(zip(("width", "heads", "kv_heads", "head_dim", "ff", "layers", "window"), SIZES[name])),
               "prefill": {"prompts": 1, "tokens": plen}, "decode": {"rows": rows, "context": ctx}}
        for spec in (postnorm_specs(name) if postnorm else parallel_specs(name) if parallel else gated_specs(name) if gated else specs(name)):
            t0 = time.perf_counter()
            ex = build(spec, rows, plen, max(plen, ctx + 256))
            tp = time_prefill(ex, 1, plen, iters)
            td = time_decode(ex, rows, ctx, 4 * iters)
            tl = time_decode(ex, rows, 64, 4 * iters)
            key = spec.family
            rec[key] = {"prefill_tok_s": round(plen / tp, 1), "prefill_ms": round(tp * 1e3, 3),
                        "decode_tok_s": round(rows / td, 1), "decode_ms": round(td * 1e3, 3),
                        "decode_short_ctx_ms": round(tl * 1e3, 3), "bringup_s": round(time.perf_counter() - t0, 1)}
            ex.drop_graphs()
            del ex
            gc.collect()
            torch.cuda.empty_cache()
        new, old = ("zovozen", "nufapel") if postnorm else ("tezesun", "letarax") if parallel else ("nufapel", "letarax") if gated else ("letarax", "llama")
        rec["prefill_ratio"] = round(rec[new]["prefill_tok_s"] / rec[old]["prefill_tok_s"], 3)
        rec["decode_ratio"] = round(rec[new]["decode_tok_s"] / rec[old]["decode_tok_s"], 3)
        out.write(json.dumps(rec) + "\n")
        out.flush()
    return 0

"""Every mechanism of the Zovozen design alone: the package's torch operations (CPU) and its HIP kernels (`gpu` marker)
against the plain float64 functions of `zovozen_oracle`, on small inputs made here."""
import pytest
import torch

import zovozen_oracle as O

F64 = torch.float64


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64) * std


def close(got, ref, tol=2e-5):
    ref = ref.to(F64)
    err = (got.detach().cpu().to(F64) - ref).abs().max().item() / max(1.0, ref.abs().max().item())
    assert err < tol, err


def attention_ref(q, k, v, scale, temp, talk, sink, chunk):
    """q [T, H, d], k [T, G, d], v [T, G, dv] as they sit in front of the scores -> [T, H, dv]."""
    H, G = q.shape[1], k.shape[1]
    p = O.sink_softmax(O.mixed_scores(q, k, scale, temp, talk), O.chunk_mask(q.shape[0], chunk), sink)
    return torch.einsum("hij,jhd->ihd", p, v.repeat_interleave(H // G, dim=1))


# ---- torch operations (the CPU executor's) ---------------------------------------------------------------------------
@pytest.mark.parametrize("H,G,d,dv,chunk", [(4, 2, 8, 12, 7), (3, 3, 6, 6, 0), (6, 1, 4, 10, 1), (2, 2, 16, 8, 32), (1, 1, 8, 8, 33)])
def test_attention_with_mixed_heads_chunks_and_sink(H, G, d, dv, chunk):
    from distributed_llm_inference_amd.ops import reference as R
    T = 70
    q, k, v = rnd(T, H, d, seed=1), rnd(T, G, d, seed=2), rnd(T, G, dv, seed=3)
    temp, talk, sink = 1.0 + rnd(H, seed=4, std=0.3), torch.eye(H, dtype=F64) + rnd(H, H, seed=5, std=0.4), rnd(H, seed=6, std=2.0)
    ref = attention_ref(q, k, v, 0.4, temp, talk, sink, chunk)
    for q0 in (0, 1, 33, 69):        # the queries of a portion that starts at q0, over the keys cached so far
        got = R.attention(q[q0:].float(), k.float(), v.float(), q0, 0.4, sink=True, temp=temp.float(), sink_logit=sink.float(),
                          chunk=chunk, head_mix=talk.float())
        close(got, ref[q0:])
    # a sink far above every score takes all the weight, one far below none
    close(R.attention(q.float(), k.float(), v.float(), 0, 0.4, sink=True, sink_logit=torch.full((H,), 60.0), chunk=chunk), torch.zeros(T, H, dv), 1e-6)
    close(R.attention(q.float(), k.float(), v.float(), 0, 0.4, sink=True, sink_logit=torch.full((H,), -60.0), chunk=chunk, temp=temp.float(), head_mix=talk.float()),
          R.attention(q.float(), k.float(), v.float(), 0, 0.4, chunk=chunk, temp=temp.float(), head_mix=talk.float()))


ROUTES = [dict(experts=6, identity=2, top=2, groups=4, keep=2), dict(experts=5, identity=0, top=1, groups=1, keep=1),
          dict(experts=4, identity=2, top=3, groups=3, keep=2), dict(experts=6, identity=0, top=2, groups=6, keep=3),
          dict(experts=10, identity=4, top=3, groups=2, keep=1), dict(experts=3, identity=1, top=4, groups=1, keep=1)]


def _router(r, H, seed, corr_std):
    outs = r["experts"] + r["identity"]
    P = {"router": rnd(outs, H, seed=seed, std=2.0 * H ** -0.5), "correction": rnd(outs, seed=seed + 1, std=corr_std)}
    return P, {"experts": r["experts"], "top": r["top"], "identity": r["identity"], "groups": {"count": r["groups"], "keep": r["keep"]}}


@pytest.mark.parametrize("r", ROUTES)
@pytest.mark.parametrize("corr_std", [0.05, 3.0])
def test_routing(r, corr_std):
    """Softmax scores, choice by score + correction (corrections of the scores' order, and so large that most choice scores
    are negative: an expert of a kept group still goes before any expert outside), groups ranked by their best member,
    weights the plain scores."""
    from distributed_llm_inference_amd.ops import reference as R
    H, T = 24, 200
    P, rc = _router(r, H, 3, corr_std)
    if corr_std > 1:
        P["correction"] = P["correction"] - 4.0
    h = rnd(T, H, seed=9)
    idx, w = O.route(h, P, rc)
    gi, gw = R.moe_route(torch.softmax((h @ P["router"].T).float(), -1), r["top"], r["groups"], r["keep"], 1.0, correction=P["correction"].float(),
                         group_rank=1, renorm=False)
    assert torch.equal(gi, idx)
    close(gw, w)


def test_matrix_memory_in_portions_and_linear_rescaling():
    from distributed_llm_inference_amd.models.rope import rope_table
    from distributed_llm_inference_amd.models.spec import RopeScaling
    from distributed_llm_inference_amd.ops import reference as R
    T, H, d, dv = 40, 3, 6, 10
    q, k, v = rnd(T, H, d, seed=1), rnd(T, H, d, seed=2), rnd(T, H, dv, seed=3)
    li, lf = rnd(T, H, seed=4, std=3.0), -torch.nn.functional.softplus(rnd(T, H, seed=5, std=2.0))
    ref = O.matrix_memory(q, k, v, li, lf)
    S, n, m, outs, t0 = torch.zeros(H, d, dv), torch.zeros(H, d), torch.zeros(H), [], 0
    for c in (1, 2, 17, 1, 19):
        o, S, n, m = R.matrix_memory(q[t0:t0 + c].float(), k[t0:t0 + c].float(), v[t0:t0 + c].float(), li[t0:t0 + c].float(), lf[t0:t0 + c].float(), S, n, m)
        outs.append(o)
        t0 += c
    close(torch.cat(outs), ref)
    # rotation of the first entries, pairs (i, i + dims / 2), frequencies divided by the factor
    x, pos = rnd(9, 2, 14, seed=6), torch.tensor([0, 1, 2, 50, 51, 52, 700, 701, 702])
    for dims, base, factor in ((14, 100.0, 1.0), (6, 500000.0, 4.0), (2, 10.0, 3.0)):
        cos, sin = rope_table(dims, base, RopeScaling(factor=factor, rope_type="linear") if factor != 1.0 else None, 710)
        close(R.rope_partial(x.float(), cos, sin, pos, False), O.rotate_half_partial(x, pos, dims, base, factor), 1e-5)


# ---- HIP kernels ------------------------------------------------------------------------------------------------------
def _K():
    from distributed_llm_inference_amd import ops
    return ops.load()


def _meta(seqs, dev):
    """seqs: [(slot, q_len, ctx)] -> tok_pos, tok_seq, q_start, ctx, slots (int32 on the device)."""
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    pos = [c + i for _, n, c in seqs for i in range(n)]
    seq = [s for s, n, _ in seqs for _ in range(n)]
    qs = [0]
    for _, n, _ in seqs:
        qs.append(qs[-1] + n)
    return i32(pos), i32(seq), i32(qs), i32([c for _, _, c in seqs]), i32([s for s, _, _ in seqs])


@pytest.mark.gpu
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_post_norm_add_hip(out_dtype):
    K, dev, T, H, eps = _K(), "cuda", 9, 200, 1e-6
    x, ya, yb, w = rnd(T, H, seed=1), rnd(T, H, seed=2, std=3.0), rnd(T, H, seed=3, std=0.2), 1.0 + rnd(H, seed=4, std=0.2)
    f = lambda t: t.float().to(dev).contiguous()
    tol = 2e-5 if out_dtype == torch.float32 else 1e-2
    for a, b, second in ((0.7, 0.6, True), (1.0, 0.0, False), (1.0, 1.0, True)):
        h, out = f(x), torch.zeros(T, H, device=dev, dtype=out_dtype)
        K.post_norm_add(out, h, f(ya), f(yb) if second else None, a, b, f(w), eps)
        ref = x + O.rms(a * ya + (b * yb if second else 0.0), eps, w)
        close(h, ref)
        close(out.float(), ref, tol)
    h, out = f(x), torch.zeros(T, H, device=dev, dtype=out_dtype)
    K.post_norm_add(out, h, None, None, 1.0, 0.0, None, eps)        # only the stream in the output's type
    close(h, x, 1e-7)
    close(out.float(), x, tol)


def _prep_and_attend(K, dev, dtype, tile, H, G, d, dv, chunk, dims, mixed, z_all, gate, P, steps, scale, eps, base, factor, direct=False):
    """Runs mix_prep + attention over `steps` ([[(slot, first token, count)]]: the sequences of every step) on a paged cache whose
    blocks are in no order; returns {slot: outputs [T, H dv]}."""
    from distributed_llm_inference_amd.models.rope import rope_table
    from distributed_llm_inference_amd.models.spec import RopeScaling
    f = lambda t: t.float().to(dev).contiguous() if t is not None else None
    cos, sin = (rope_table(dims, base, RopeScaling(factor=factor, rope_type="linear") if factor != 1.0 else None, 400, dev) if dims else (None, None))
    kd, gk = (G * d, 1) if mixed else (d, G)
    nblk = 12
    kc = torch.zeros(nblk, gk, 32, G * d // gk, device=dev, dtype=dtype)
    vc = torch.zeros(nblk, G, dv, 32, device=dev, dtype=dtype) if tile else torch.zeros(nblk, G, 32, dv, device=dev, dtype=dtype)
    table = torch.full((3, 6), -1, dtype=torch.int32, device=dev)
    table[1, :5] = torch.tensor([7, 2, 5, 0, 3], dtype=torch.int32)
    table[2, :5] = torch.tensor([11, 1, 9, 4, 6], dtype=torch.int32)
    mix = f(P["talk"] * P["temp"].view(1, -1) * scale) if mixed else None
    got = {}
    for step in steps:
        tok_pos, tok_seq, q_start, ctx, slots = _meta([(s, n, t0) for s, t0, n in step], dev)
        z = f(torch.cat([z_all[t0:t0 + n] for _, t0, n in step]))
        gt = f(torch.cat([gate[t0:t0 + n] for _, t0, n in step]))
        T = z.shape[0]
        out = torch.zeros(T, H * dv, device=dev, dtype=dtype)
        qf = torch.zeros(T, H * kd, device=dev, dtype=dtype if tile else torch.float32)
        if direct and max(n for _, _, n in step) > 1:      # plain queries, the mix applied to the finished score tiles
            q16 = torch.zeros(T, H * d, device=dev, dtype=dtype)
            K.mix_prep(z, H, G, d, dv, f(P["q.norm"]), f(P["k.norm"]), eps, dims, cos, sin, True, None, q16, kc, vc, True, tok_pos, tok_seq, table)
            part = torch.zeros(int(K.mixed_attention_part_floats(T, H, dv)), device=dev) if T > 60 else None      # (with it a tile's key blocks go to several workgroups)
            K.mixed_attention(out, q16, kc, vc, mix, q_start, ctx, slots, table, max(n for _, _, n in step), H, d, dv, chunk, f(P["sink"]), gt, part)
        else:
            K.mix_prep(z, H, G, d, dv, f(P["q.norm"]), f(P["k.norm"]), eps, dims, cos, sin, True, mix, qf, kc, vc, tile, tok_pos, tok_seq, table)
        if direct and max(n for _, _, n in step) > 1:
            pass
        elif tile:
            part = torch.zeros(int(K.tile_attention_part_floats(len(step), H, G, dv, 1, gk)), device=dev)
            K.tile_attention(out, qf, kd, kc, vc, q_start, ctx, slots, table, max(n for _, _, n in step), H, kd, dv, 1, 1.0 if mixed else scale,
                             0, 0, 0.0, 0.0, 1.0, eps, gt, part, chunk, f(P["sink"]))
        else:
            K.multi_attention(out, qf, kd, kc, vc, 0, tok_pos, tok_seq, table, H, kd, dv, 1, 1.0 if mixed else scale, 0, 0, 0.0, 0.0, 1.0, eps,
                              gt, chunk, f(P["sink"]))
        r = 0
        for s, _, n in step:
            got.setdefault(s, []).append(out[r:r + n].float().cpu())
            r += n
    return {s: torch.cat(v) for s, v in got.items()}


def _attention_case(H, G, d, dv, dims, mixed, seed=1):
    T, eps, scale, base, factor = 150, 1e-5, 0.3, 50.0, 2.0
    z_all = torch.cat([rnd(T, H * d, seed=seed), rnd(T, G * d, seed=seed + 1), rnd(T, G * dv, seed=seed + 2, std=2.0)], 1)
    gate = rnd(T, H * dv, seed=seed + 3)
    P = {"q.norm": 1.0 + rnd(H * d, seed=seed + 4, std=0.2), "k.norm": 1.0 + rnd(G * d, seed=seed + 5, std=0.2),
         "temp": (1.0 + rnd(H, seed=seed + 6, std=0.3)) if mixed else torch.ones(H, dtype=F64),
         "talk": (torch.eye(H, dtype=F64) + rnd(H, H, seed=seed + 7, std=0.4)) if mixed else torch.eye(H, dtype=F64),
         "sink": rnd(H, seed=seed + 8, std=1.5)}
    return T, eps, scale, base, factor, z_all, gate, P


def _attention_oracle(T, H, G, d, dv, chunk, dims, z_all, gate, P, scale, eps, base, factor, round_bf16=False):
    q, k, v = z_all[:, :H * d], z_all[:, H * d:(H + G) * d], z_all[:, (H + G) * d:]
    q, k = O.rms(q, eps, P["q.norm"]).view(T, H, d), O.rms(k, eps, P["k.norm"]).view(T, G, d)
    pos = torch.arange(T)
    q, k = O.rotate_half_partial(q, pos, dims, base, factor), O.rotate_half_partial(k, pos, dims, base, factor)
    v = O.rms(v.view(T, G, dv), eps)
    if round_bf16:       # (what the cache holds)
        k, v = k.bfloat16().to(F64), v.bfloat16().to(F64)
    return attention_ref(q, k, v, scale, P["temp"], P["talk"], P["sink"], chunk).reshape(T, H * dv) * torch.sigmoid(gate)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,chunk,dims,mixed", [
    (4, 2, 16, 24, 40, 8, True), (2, 1, 8, 8, 0, 8, True), (3, 3, 12, 70, 33, 4, True), (2, 2, 72, 130, 32, 0, False),
    (6, 1, 10, 16, 64, 10, True), (6, 3, 10, 6, 1, 2, True), (4, 2, 16, 24, 97, 16, False)])
def test_preparation_cache_write_and_attention_hip(dtype, H, G, d, dv, chunk, dims, mixed):
    """mix_prep (whole-projection norms, rotation, unit values, the head mix folded into the query, cache write) + the
    one-wave-per-(token, head) attention with chunked mask, sink and gate: a prompt portion, another that crosses block and
    chunk edges, single tokens, against whole-sequence attention."""
    K, dev = _K(), "cuda"
    T, eps, scale, base, factor, z_all, gate, P = _attention_case(H, G, d, dv, dims, mixed)
    ref = _attention_oracle(T, H, G, d, dv, chunk, dims, z_all, gate, P, scale, eps, base, factor, dtype == torch.bfloat16)
    steps, t0 = [], 0
    for n in (50, 47, 1, 1, 1, 50):
        steps.append([(1, t0, n)])
        t0 += n
    got = _prep_and_attend(K, dev, dtype, False, H, G, d, dv, chunk, dims, mixed, z_all, gate, P, steps, scale, eps, base, factor)
    close(got[1], ref, 2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,dv,chunk,dims,mixed", [
    (4, 2, 16, 24, 40, 8, True), (2, 1, 8, 8, 0, 8, True), (3, 3, 24, 70, 33, 4, True), (2, 2, 72, 130, 32, 0, False),
    (6, 1, 40, 16, 64, 10, True), (8, 2, 32, 300, 1, 16, True), (4, 4, 64, 80, 96, 32, True), (16, 4, 8, 8, 50, 8, True),
    (16, 8, 16, 24, 50, 8, True), (12, 6, 8, 16, 0, 4, True), (40, 8, 8, 8, 70, 8, True)])     # (many value heads: tiles of 16 heads)
def test_matrix_core_attention_hip(H, G, d, dv, chunk, dims, mixed):
    """The same through the matrix-core kernel (bf16, values key-contiguous in the cache) on two sequences that share steps
    with different portions (down to single tokens; one step of single tokens only, whose key blocks are dealt out to
    workgroups and merged with the sink), blocks in no order."""
    K, dev = _K(), "cuda"
    T, eps, scale, base, factor, z_all, gate, P = _attention_case(H, G, d, dv, dims, mixed, seed=11)
    ref = _attention_oracle(T, H, G, d, dv, chunk, dims, z_all, gate, P, scale, eps, base, factor, True)
    steps, a0, b0 = [], 0, 0
    for na, nb in zip((50, 47, 1, 1, 1, 50), (1, 20, 30, 1, 34, 64)):
        steps.append([(2, b0, nb), (1, a0, na)])
        a0, b0 = a0 + na, b0 + nb
    got = _prep_and_attend(K, dev, torch.bfloat16, True, H, G, d, dv, chunk, dims, mixed, z_all, gate, P, steps, scale, eps, base, factor)
    close(got[1], ref, 3e-2)
    close(got[2], ref, 3e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,d,dv,chunk,dims", [
    (4, 2, 16, 24, 40, 8), (2, 1, 8, 8, 0, 8), (3, 3, 24, 70, 33, 4), (6, 1, 40, 16, 64, 10), (8, 2, 32, 128, 1, 16), (4, 4, 64, 80, 96, 32),
    (16, 4, 128, 128, 50, 64), (32, 8, 64, 64, 70, 32), (24, 6, 8, 8, 0, 8), (17, 17, 16, 16, 45, 0), (2, 2, 256, 104, 31, 128)])
def test_mixed_score_tiles_attention_hip(H, G, d, dv, chunk, dims):
    """The prompt-step kernel that mixes the finished score tiles (plain queries; up to 16 heads one workgroup per 16 tokens,
    beyond that two that share the output heads) beside the single-token steps through the query that carries the mix: two
    sequences with different portions in one step, blocks in no order, against whole-sequence attention."""
    K, dev = _K(), "cuda"
    assert K.mixed_attention_fits(H, G, d, dv)
    T, eps, scale, base, factor, z_all, gate, P = _attention_case(H, G, d, dv, dims, True, seed=21)
    ref = _attention_oracle(T, H, G, d, dv, chunk, dims, z_all, gate, P, scale, eps, base, factor, True)
    steps, a0, b0 = [], 0, 0
    for na, nb in zip((50, 47, 1, 1, 1, 50), (1, 20, 30, 1, 34, 64)):
        steps.append([(2, b0, nb), (1, a0, na)])
        a0, b0 = a0 + na, b0 + nb
    got = _prep_and_attend(K, dev, torch.bfloat16, True, H, G, d, dv, chunk, dims, True, z_all, gate, P, steps, scale, eps, base, factor, direct=True)
    close(got[1], ref, 3e-2)
    close(got[2], ref, 3e-2)
    assert not K.mixed_attention_fits(40, 8, 16, 16) and not K.mixed_attention_fits(4, 2, 12, 16) and not K.mixed_attention_fits(4, 2, 16, 136)


@pytest.mark.gpu
@pytest.mark.parametrize("r", ROUTES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routed_feed_forward_hip(r, dtype):
    """route -> plan -> the experts' GEMMs over sorted rows -> weighted sum with the identity experts' share of the input, and
    the shared expert's activation, against the plain feed-forward (the router's choice against the plain routing)."""
    K, dev = _K(), "cuda"
    H, T, ff = 32, 75, 24
    P, rc = _router(r, H, 3, 0.05)
    E, outs = r["experts"], r["experts"] + r["identity"]
    for e in range(E):
        P[f"e{e}.gate"], P[f"e{e}.up"], P[f"e{e}.down"] = rnd(ff, H, seed=20 + e, std=H ** -0.5), rnd(ff, H, seed=40 + e, std=H ** -0.5), rnd(H, ff, seed=60 + e, std=ff ** -0.5)
    h = rnd(T, H, seed=9)
    if dtype == torch.bfloat16:
        P = {k: v.bfloat16().to(F64) for k, v in P.items()}
        h = h.bfloat16().to(F64)
    ref = O.moe_ff(h, P, {"router": rc})
    idx, w = O.route(h, P, rc)
    f = lambda t: t.float().to(dev).contiguous()
    top = r["top"]
    sel, wts = torch.zeros(T * top, dtype=torch.int32, device=dev), torch.zeros(T * top, device=dev)
    K.moe_route(sel, wts, f(h @ P["router"].T), top, r["groups"], r["keep"], 1.0, f(P["correction"]), True, 1, False)
    assert torch.equal(sel.view(T, top).cpu().long(), idx)
    close(wts.view(T, top), w)
    nt = (T * top + 31) // 32 + E
    tiles, row_tok, pair_row = (torch.zeros(n, dtype=torch.int32, device=dev) for n in (1 + nt, 32 * nt, T * top))
    x = f(h).to(dtype)
    stack = lambda n: torch.stack([P[f"e{e}.{n}"] for e in range(E)]).float().to(dev).to(dtype).contiguous()
    eact, ey, out = torch.zeros(32 * nt, ff, device=dev, dtype=dtype), torch.zeros(32 * nt, H, device=dev), torch.zeros(T, H, device=dev)
    K.moe_plan(tiles, row_tok, pair_row, sel, T * top, top, E, 32)
    K.moe_up(eact, x, stack("gate"), stack("up"), tiles, row_tok, nt, 0.0, 32)
    K.moe_down(ey, eact, stack("down"), tiles, row_tok, nt, 32)
    K.moe_combine(out, ey, pair_row, wts, top, f(h))
    close(out, ref, 2e-5 if dtype == torch.float32 else 2e-2)
    assert ((pair_row.view(T, top).cpu() < 0) == (idx >= E)).all()
    # squared relu, and silu(gate) * up from gate | up side by side
    z = rnd(T, 2 * ff, seed=5, std=2.0)
    act = torch.zeros(T, ff, device=dev, dtype=dtype)
    K.unary_act(act, f(z)[:, :ff], 2)
    close(act.float(), torch.relu(z[:, :ff]) ** 2, 2e-5 if dtype == torch.float32 else 1e-2)
    K.unary_act(act, f(z), 3)
    close(act.float(), z[:, :ff] * torch.sigmoid(z[:, :ff]) * z[:, ff:], 2e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("H,d,dv,cap", [(3, 6, 10, 12.0), (1, 32, 64, 6.0), (4, 16, 8, 30.0)])
def test_matrix_memory_branch_hip(H, d, dv, cap):
    """Gates from their logits and biases (capped, log-sigmoid), the recurrence from a slot that held another sequence, the
    read-out's division, per-head norm, weight and gate: two sequences over three steps against the plain branch."""
    K, dev, W, eps = _K(), "cuda", 20, 1e-5
    P = {"q": rnd(H * d, W, seed=1, std=W ** -0.5), "k": rnd(H * d, W, seed=2, std=W ** -0.5), "v": rnd(H * dv, W, seed=3, std=W ** -0.5),
         "g": rnd(H * dv, W, seed=4, std=W ** -0.5), "i": rnd(H, W, seed=5, std=3.0 * W ** -0.5), "i.b": rnd(H, seed=6),
         "f": rnd(H, W, seed=7, std=3.0 * W ** -0.5), "f.b": rnd(H, seed=8) + 2.0, "norm": 1.0 + rnd(H * dv, seed=9, std=0.1),
         "o": torch.eye(H * dv, dtype=F64)}
    c = {"heads": H, "dim": d, "vdim": dv, "gate_cap": cap}
    xa, xb = rnd(45, W, seed=10), rnd(30, W, seed=11)
    refs = {1: O.right_memory(xa, P, c, eps), 3: O.right_memory(xb, P, c, eps)}
    f = lambda t: t.float().to(dev).contiguous()
    w_in = torch.cat([P[n] for n in ("q", "k", "v", "g", "i", "f")])
    state, mstate = torch.full((5, H, d, dv + 1), 3.0, device=dev), torch.full((5, H, 128), 2.0, device=dev)      # stale slots
    b_if = f(torch.cat([P["i.b"], P["f.b"]]))
    c_k, c_v, c_g, c_i, c_f = H * d, 2 * H * d, 2 * H * d + H * dv, 2 * H * d + 2 * H * dv, 2 * H * d + 2 * H * dv + H
    got, a0, b0 = {1: [], 3: []}, 0, 0
    for na, nb in ((20, 1), (1, 1), (24, 28)):
        _, _, q_start, ctx, slots = _meta([(1, na, a0), (3, nb, b0)], dev)
        z = f(torch.cat([xa[a0:a0 + na], xb[b0:b0 + nb]]) @ w_in.T)
        T = na + nb
        o, out = torch.zeros(T, H * (dv + 2), device=dev), torch.zeros(T, H * dv, device=dev)
        K.state_scan(1, o, z, None, state, mstate, b_if, None, q_start, ctx, slots, H, d, dv, 0, c_k, c_v, 0, c_i, c_f, cap, d ** -0.5, max(na, nb), False)
        K.headnorm_gate(out, o, z[:, c_g:c_g + H * dv], f(P["norm"]), H, dv, 2, eps)
        got[1].append(out[:na].cpu())
        got[3].append(out[na:].cpu())
        a0, b0 = a0 + na, b0 + nb
    close(torch.cat(got[1]), refs[1], 5e-5)
    close(torch.cat(got[3]), refs[3], 5e-5)

"""The Rigulorn design (differential attention, selective state-space mixer, residual streams, clamped gated unit)
on the GPU against the plain CPU implementation in oracle/rigulorn.py.

Every test makes its own small configuration and random weights. fp32 weights are compared tightly (the kernels then
run plain fp32); bf16 weights within the noise of bf16 operands. Schedules (whole prompt, token by token, portions,
batches, reused slots) must not change a position's logits beyond rounding. Where random weights would hide a fault
(a key far back, a chunk's edge) the operation is called on crafted inputs in which one score stands out.
"""

from pathlib import Path

import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import rigulorn as orc  # noqa: E402


# ------------------------------------------------------------------------------------------------ configurations
def att(heads=2, kv_heads=None, dim=8, vdim=12, rot_dims=None, base=500.0, diff=0.4, softcap=8.0, mask=5, scale=None,
        kv_from=None):
    m = {"heads": heads, "kv_heads": heads if kv_heads is None else kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
         "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base},
         "scale": dim ** -0.5 if scale is None else scale}
    if softcap:
        m["softcap"] = softcap
    if mask:
        m["mask"] = {"size": mask}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def ssm(heads=4, vdim=6, state=8, groups=2, norm_groups=2, conv=3):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
                                        "norm_groups": norm_groups, "conv": conv}}


def dense(ff=40, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def make_cfg(layers, width=40, vocab=53, streams=2, eps=1e-5, emb_scale=3.0):
    cfg = {"architecture": "Rigulorn", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": emb_scale}, "layers": [dict(l[0], mlp=l[1]) for l in layers]}
    if streams:
        cfg["streams"] = streams
    return cfg


MIXED = [(ssm(), None), (att(heads=4, kv_heads=2), dense()), (att(heads=4, kv_heads=2, mask=7, kv_from=1), dense(24, 0.7)),
         (ssm(heads=3, vdim=10, state=12, groups=1, norm_groups=3, conv=5), dense()), (att(heads=3, kv_heads=1, rot_dims=4), None)]


def build(cfg, dtype=torch.float32, seed=0, edit=None):
    from lit_gpt.config import LayeredConfig
    from lit_gpt.layered import LayeredGPT

    config = LayeredConfig.from_dict(cfg)
    weights = LayeredGPT.random_weights(config, seed=seed)
    if edit:
        edit(weights)
    model = LayeredGPT(config, weights, device=torch.device("cuda", 0), dtype=dtype)
    return model, weights


def tokens_of(n, vocab, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rel_err(got, want):
    """Per row: rms of the mean-free difference over the rms of the mean-free reference."""
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def engine_logits(model, seqs, cuts, max_seq=None, engine=None):
    """Run sequences together through the BatchEngine: ``cuts[i]`` lists how many tokens request i brings per step
    (0: it sits the step out). Returns the logits of every position per request."""
    from generate.batch import BatchEngine

    eng = engine or BatchEngine(model, max_seq_length=max_seq or max(len(s) for s in seqs), slots=1)
    out = [[] for _ in seqs]
    at = [0] * len(seqs)
    ids = [object() for _ in seqs]
    for step in range(max(len(c) for c in cuts)):
        entries, who, end = [], [], []
        for i, s in enumerate(seqs):
            n = cuts[i][step] if step < len(cuts[i]) else 0
            if n:
                entries.append((ids[i], s[at[i]:at[i] + n], list(range(n))))
                who.append((i, n))
                at[i] += n
                if at[i] == len(s):
                    end.append(ids[i])
        lg = eng.step(entries, end)
        row = 0
        for i, n in who:
            out[i].append(lg[row:row + n].cpu())
            row += n
    assert all(a == len(s) for a, s in zip(at, seqs))
    return [torch.cat(o) for o in out]


def portions(n, size):
    return [size] * (n // size) + ([n % size] if n % size else [])


TOL32, TOL16, SAME = 2e-4, 6e-2, 2e-5


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("layers,streams", [
    ([(att(), None)], 0),
    ([(att(heads=4, kv_heads=2, dim=6, vdim=10, rot_dims=2, mask=3), None)], 0),  # key size no multiple of 4
    ([(att(heads=3, kv_heads=1, dim=12, vdim=72, rot_dims=0, softcap=0, mask=0), None)], 0),  # no cap, mask, rotation
    ([(att(heads=1, dim=16, vdim=136, mask=1), None)], 0),  # every query sees itself only; 256 value columns
    ([(att(heads=2, dim=20, vdim=8, mask=64, diff=0.0), None)], 0),  # one chunk holds the whole sequence
    ([(ssm(), None)], 0),
    ([(ssm(heads=2, vdim=72, state=40, groups=2, norm_groups=1, conv=1), None)], 0),  # two column blocks, no history
    ([(ssm(heads=6, vdim=4, state=100, groups=3, norm_groups=6, conv=7), None)], 0),
    ([(ssm(heads=1, vdim=8, state=130, groups=1, norm_groups=4, conv=2), None)], 0),
    ([(att(), dense())], 0),
    ([(att(), dense(ff=33, limit=0.3))], 0),  # most gates and ups are clamped
    ([(att(), dense())], 1),
    ([(ssm(), dense())], 3),
    ([(att(), dense()), (ssm(), None)], 4),
    ([(att(heads=2, mask=4), None), (ssm(), None), (att(heads=2, mask=9, kv_from=0), dense())], 2),  # another mask
])
def test_mechanism_against_plain(layers, streams):
    cfg = make_cfg(layers, streams=streams)
    model, w = build(cfg)
    toks = tokens_of(29, cfg["vocab"])
    want = orc.forward(cfg, w, toks)
    got = engine_logits(model, [toks], [[len(toks)]])[0]
    assert rel_err(got, want).max() < TOL32
    got = engine_logits(model, [toks], [[1] * len(toks)])[0]
    assert rel_err(got, want).max() < TOL32


def test_streams_after_every_layer():
    from lit_gpt.mixers import StepBatch

    cfg = make_cfg(MIXED, streams=3)
    model, w = build(cfg)
    toks = tokens_of(23, cfg["vocab"])
    want = []
    orc.forward(cfg, w, toks, layers_out=want)
    model.set_kv_cache(1, 32)
    got = []
    with torch.inference_mode():
        model._forward_streams(StepBatch.build([(0, 0, toks)], model.device),
                               after_layer=lambda run, x: got.append(x.sum(1).cpu()))
    assert len(got) == len(want) == len(MIXED)
    for g, e in zip(got, want):
        assert (g.double() - e).abs().max() < 1e-4 * e.abs().max()


@pytest.mark.parametrize("width,vocab", [(8, 11), (50, 300), (136, 70)])
def test_other_widths(width, vocab):
    cfg = make_cfg(MIXED, width=width, vocab=vocab, streams=3)
    model, w = build(cfg, seed=3)
    toks = tokens_of(21, vocab, seed=2)
    assert rel_err(engine_logits(model, [toks], [[len(toks)]])[0], orc.forward(cfg, w, toks)).max() < TOL32


def test_bf16_within_operand_noise():
    cfg = make_cfg(MIXED, streams=3)
    model, w = build(cfg, dtype=torch.bfloat16)
    toks = tokens_of(40, cfg["vocab"])
    want = orc.forward(cfg, w, toks)
    whole = engine_logits(model, [toks], [[len(toks)]])[0]
    single = engine_logits(model, [toks], [[24] + [1] * 16])[0]
    assert rel_err(whole, want).max() < TOL16
    assert rel_err(single, want).max() < TOL16


# ------------------------------------------------------------------------------------------------ schedules
def slow_state(w):
    for k in w:
        if k.endswith("A_log"):
            w[k] = torch.full_like(w[k], -20.0)  # decay exp(-exp(-20) dt) = 1: what the state took in stays


@pytest.mark.parametrize("edit", [None, slow_state])
def test_prompt_portions_and_single_tokens_agree(edit):
    cfg = make_cfg(MIXED, streams=3)
    model, w = build(cfg, edit=edit)
    n = 45
    toks = tokens_of(n, cfg["vocab"], seed=5)
    want = orc.forward(cfg, w, toks)
    whole = engine_logits(model, [toks], [[n]])[0]
    assert rel_err(whole, want).max() < TOL32
    for cuts in ([1] * n, portions(n, 2), portions(n, 3), portions(n, 7), portions(n, 16), [17, 1, 1, 2, 24],
                 [30] + [1] * 15):
        got = engine_logits(model, [toks], [cuts])[0]
        assert rel_err(got, whole).max() < SAME, cuts


def test_unequal_batch_equals_each_alone():
    cfg = make_cfg(MIXED, streams=2)
    model, w = build(cfg, seed=1)
    lens = [1, 37, 9, 22]
    seqs = [tokens_of(n, cfg["vocab"], seed=i) for i, n in enumerate(lens)]
    alone = [engine_logits(model, [s], [[len(s)]])[0] for s in seqs]
    # prompts of unequal lengths in one step (all but the last 4 tokens), then decoded together; shorter ones end earlier
    cuts = [[max(1, n - 4)] + [1] * (n - max(1, n - 4)) for n in lens]
    together = engine_logits(model, seqs, cuts, max_seq=40)
    for a, b in zip(alone, together):
        assert rel_err(b, a).max() < SAME
    assert rel_err(alone[1], orc.forward(cfg, w, seqs[1])).max() < TOL32


def test_slots_freed_reused_and_grown():
    from generate.batch import BatchEngine

    cfg = make_cfg(MIXED, streams=2)
    model, w = build(cfg, seed=2)
    a, b, c, d = (tokens_of(n, cfg["vocab"], seed=10 + n) for n in (33, 12, 27, 18))
    ref = {id(s): engine_logits(model, [s], [[len(s)]])[0] for s in (a, b, c, d)}
    eng = BatchEngine(model, max_seq_length=40, slots=1)
    # a fills slot 0 with a long sequence and ends; b takes the same slot and must not see what a left
    got_a = engine_logits(model, [a], [[20, 13]], engine=eng)[0]
    got_b = engine_logits(model, [b], [[5] + [1] * 7], engine=eng)[0]
    assert eng.pool.size == 1
    assert rel_err(got_a, ref[id(a)]).max() < SAME and rel_err(got_b, ref[id(b)]).max() < SAME
    # three at once: the caches grow while c is in flight
    lg_c0 = eng.step([("c", c[:10], list(range(10)))])
    both = eng.step([("c", c[10:], list(range(17))), ("d", d, list(range(18))), ("a", a, list(range(33)))],
                    end=["c", "d", "a"])
    got_c = torch.cat([lg_c0.cpu(), both[:17].cpu()])
    assert model.slots >= 3
    assert rel_err(got_c, ref[id(c)]).max() < SAME
    assert rel_err(both[17:35], ref[id(d)]).max() < SAME
    assert rel_err(both[35:], ref[id(a)]).max() < SAME


def test_first_token_alone_and_long_decoding():
    cfg = make_cfg([(ssm(), None), (att(heads=2, mask=50), dense()), (att(heads=2, mask=16, kv_from=1), None)], streams=2)
    model, w = build(cfg, seed=4)
    n = 230
    toks = tokens_of(n, cfg["vocab"], seed=8)
    whole = engine_logits(model, [toks], [[n]])[0]
    single = engine_logits(model, [toks], [[1] * n])[0]
    assert rel_err(single, whole).max() < SAME
    short = orc.forward(cfg, w, toks[:60])
    assert rel_err(single[:60], short).max() < TOL32
    first = engine_logits(model, [toks[:1]], [[1]])[0]
    assert rel_err(first, short[:1]).max() < TOL32


# ------------------------------------------------------------------------------------------------ crafted attention
def plain_diffattn(q, k, v, pos_q, chunk, scale, cap, lam, eps, post, group):
    """q (n, H, 2, d) rotated queries at positions pos_q of one sequence whose cache holds k (S, G, 2, d), v (S, G, dv)."""
    n, H = q.shape[:2]
    out = torch.zeros(n, H, v.shape[-1], dtype=torch.float64)
    for i in range(n):
        p = pos_q[i]
        lo = p - p % chunk if chunk else 0
        for h in range(H):
            g = h // group
            a = []
            for m in range(2):
                s = (k[lo:p + 1, g, m].double() @ q[i, h, m].double()) * scale
                if cap:
                    s = cap * torch.tanh(s / cap)
                a.append(torch.softmax(s, 0) @ v[lo:p + 1, g].double())
            o = a[0] - lam * a[1]
            out[i, h] = o / torch.sqrt((o * o).mean() + eps) * post
    return out.reshape(n, -1)


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk,S", [(0, 700), (64, 300), (256, 600), (257, 600)])
def test_attention_far_keys_and_chunk_edges(chunk, S, cache_dtype):
    """One key per probe is made to dominate map 1 (its value is then the head's output before the difference): the
    chunk's first key (just inside), the key before it (just outside), a key far back, at a key-tile border (256),
    and the query's own. Prompt rows (8-query tiles that straddle a chunk edge) and one-token steps, also split."""
    from lit_gpt import seq_ops
    from lit_gpt.mixers import StepBatch

    dev = torch.device("cuda", 0)
    H, G, d, dv = 4, 2, 16, 24
    g = torch.Generator().manual_seed(chunk + S)
    k = torch.randn(S, G, 2, d, generator=g) * 0.3
    v = torch.randn(S, G, dv, generator=g)
    nq = 21
    p0 = S - nq
    q = torch.randn(nq, H, 2, d, generator=g) * 0.3
    pos_q = list(range(p0, S))
    for i in range(nq):  # query i's map 1 of head i % H points at one chosen key
        p = pos_q[i]
        lo = p - p % chunk if chunk else 0
        target = [lo, max(lo - 1, 0), max(lo, p - 256), max(lo, p - 255), p, (lo + p) // 2, 0][i % 7]
        gsel = (i % H) // (H // G)
        q[i, i % H, 0] = 25.0 * k[target, gsel, 0] / k[target, gsel, 0].norm() ** 2
    if cache_dtype == torch.bfloat16:
        k, v = k.bfloat16().float(), v.bfloat16().float()
    want = plain_diffattn(q, k, v, pos_q, chunk, 1.0, 30.0, 0.3, 1e-6, 0.8, H // G)
    ck = torch.zeros(2, S, G, 2 * d, dtype=cache_dtype, device=dev)
    cv = torch.zeros(2, S, G, dv, dtype=cache_dtype, device=dev)
    ck[1] = k.reshape(S, G, 2 * d).to(dev, cache_dtype)
    cv[1] = v.to(dev, cache_dtype)
    ck[0].fill_(7.0)  # another sequence's slot: never read
    kw = dict(H=H, G=G, d=d, dv=dv, chunk=chunk, scale=1.0, cap=30.0, lam=0.3, eps=1e-6, post=0.8)
    proj = q.reshape(nq, -1).to(dev).contiguous()
    step = StepBatch.build([(1, p0, [0] * nq)], dev)
    got = seq_ops.diffattn(proj, 0, ck, cv, step.seq_start, step.seq_slot, step.seq_pos0, nq, **kw)
    assert (got.double().cpu() - want).abs().max() < 2e-4
    for i in (0, 1, 2, 3, 4, nq - 1):  # one-token steps, whole and split over the keys
        one = StepBatch.build([(1, pos_q[i], [0])], dev)
        for splits in (1, 3, None):
            got = seq_ops.diffattn(proj[i:i + 1].contiguous(), 0, ck, cv, one.seq_start, one.seq_slot, one.seq_pos0, 1,
                                   splits=splits, **kw)
            assert (got.double().cpu() - want[i]).abs().max() < 2e-4, (i, splits)


def test_keys_rotate_by_their_own_position():
    """A layer whose scores depend on positions only through the rotation: with q = k direction and base 1 the score
    of a key at distance n is cos(n) * |.|^2; decode far from the start must match the prompt form and the oracle."""
    cfg = make_cfg([(att(heads=1, dim=2, vdim=4, base=1.0, softcap=0, mask=0, scale=3.0), None)], streams=0)
    model, w = build(cfg, seed=6)
    toks = tokens_of(90, cfg["vocab"], seed=3)
    want = orc.forward(cfg, w, toks)
    assert rel_err(engine_logits(model, [toks], [[70] + [1] * 20])[0], want).max() < TOL32


# ------------------------------------------------------------------------------------------------ crafted state
@pytest.mark.parametrize("taps", [2, 4, 9])
def test_convolution_history_across_steps(taps):
    """The convolution's inputs before a step come from the slot's stored history: portions shorter than the history,
    a slot with another sequence's history, and a sequence that restarts at position 0 (history counts as zero)."""
    from lit_gpt import seq_ops
    from lit_gpt.mixers import StepBatch

    dev = torch.device("cuda", 0)
    C, n = 70, 40
    g = torch.Generator().manual_seed(taps)
    u = torch.randn(n, C + 3, generator=g)
    wgt, bias = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    want = orc.silu(orc.causal_conv(u[:, 3:].double(), wgt.double(), bias.double()))
    state = torch.full((3, taps - 1, C), 5.0, device=dev)  # stale contents everywhere
    for cuts in ([n], [1] * n, [2, 1, 3, 1, 1, 17, 15], portions(n, taps - 1 or 1)):
        at, outs = 0, []
        for c in cuts:
            step = StepBatch.build([(2, at, [0] * c)], dev)
            outs.append(seq_ops.conv_silu(u[at:at + c].to(dev).contiguous(), 3, wgt.to(dev), bias.to(dev), state,
                                          step.seq_start, step.seq_slot, step.seq_pos0, c))
            at += c
        assert (torch.cat(outs).double().cpu() - want).abs().max() < 1e-5, cuts
    assert (state[:2] == 5.0).all()


def test_state_carries_a_far_token():
    """With a decay of one and a step size that is large at one early token only, the output late in the sequence is
    dominated by that token; every schedule must carry it."""
    def edit(w):
        slow_state(w)
        for k in w:
            if k.endswith("dt_bias"):
                w[k] = torch.full_like(w[k], -6.0)

    cfg = make_cfg([(ssm(heads=2, vdim=8, state=16, groups=1, norm_groups=1, conv=2), None)], streams=0)
    model, w = build(cfg, edit=edit, seed=9)
    n = 150
    toks = tokens_of(n, cfg["vocab"], seed=4)
    want = orc.forward(cfg, w, toks[:50])
    whole = engine_logits(model, [toks], [[n]])[0]
    assert rel_err(whole[:50], want).max() < TOL32
    for cuts in ([1] * n, portions(n, 8), portions(n, 9), [3] + [1] * 147):
        assert rel_err(engine_logits(model, [toks], [cuts])[0], whole).max() < SAME


def plain_scan(xbc, dt_raw, dt_bias, A_log, D, heads, groups, N, dv, S0):
    """Token by token in float64; returns y (T, heads dv) and the final state (heads, N, dv)."""
    T = xbc.shape[0]
    inner = heads * dv
    x = xbc[:, :inner].double().view(T, heads, dv)
    Bm = xbc[:, inner:inner + groups * N].double().view(T, groups, N)
    Cm = xbc[:, inner + groups * N:].double().view(T, groups, N)
    dt = orc.softplus(dt_raw.double() + dt_bias.double())
    a = torch.exp(-torch.exp(A_log.double()) * dt)
    S = S0.double().clone()
    y = torch.zeros(T, heads, dv, dtype=torch.float64)
    for t in range(T):
        for h in range(heads):
            g = h // (heads // groups)
            S[h] = a[t, h] * S[h] + dt[t, h] * torch.outer(Bm[t, g], x[t, h])
            y[t, h] = S[h].T @ Cm[t, g] + D[h].double() * x[t, h]
    return y.reshape(T, inner), S


@pytest.mark.parametrize("heads,groups,N,dv", [(4, 2, 16, 8), (2, 1, 40, 70), (3, 3, 128, 64), (2, 2, 5, 3)])
def test_scan_prompt_form_against_token_walk(heads, groups, N, dv):
    """Several sequences of unequal lengths (one chunk, several chunks, a chunk's edge) in one step, continued from a
    state in the slot or started anew over a slot with stale contents; both forms against float64."""
    from lit_gpt import seq_ops
    from lit_gpt.mixers import StepBatch

    dev = torch.device("cuda", 0)
    g = torch.Generator().manual_seed(N + dv)
    lens, pos0 = [64, 150, 17, 65, 1], [0, 9, 3, 0, 7]
    T, inner = sum(lens), heads * dv
    xbc = torch.randn(T, inner + 2 * groups * N, generator=g) * 0.5
    raw = torch.randn(T, heads + 2, generator=g)
    dt_bias, A_log, D = torch.randn(heads, generator=g) - 1.0, torch.randn(heads, generator=g), torch.randn(heads, generator=g)
    stale = torch.randn(len(lens) + 1, heads, N, dv, generator=g)
    want_y, want_s, at = [], [], 0
    for i, (n, p0) in enumerate(zip(lens, pos0)):
        S0 = stale[i] if p0 > 0 else torch.zeros(heads, N, dv)
        y, S = plain_scan(xbc[at:at + n], raw[at:at + n, 2:], dt_bias, A_log, D, heads, groups, N, dv, S0)
        want_y.append(y)
        want_s.append(S)
        at += n
    want_y = torch.cat(want_y)
    step = StepBatch.build([(i, p0, [0] * n) for i, (n, p0) in enumerate(zip(lens, pos0))], dev)
    for chunked in (False, True):
        state = stale.to(dev).clone()
        y = seq_ops.ssm_scan(xbc.to(dev), raw.to(dev), 2, dt_bias.to(dev), A_log.to(dev), D.to(dev), state,
                             step.seq_start, step.seq_slot, step.seq_pos0, heads=heads, groups=groups, N=N, dv=dv,
                             max_len=max(lens), chunked=chunked)
        scale = want_y.abs().max()
        assert (y.double().cpu() - want_y).abs().max() < 2e-5 * scale, chunked
        for i, S in enumerate(want_s):
            assert (state[i].double().cpu() - S).abs().max() < 2e-5 * S.abs().max().clamp_min(1.0), (chunked, i)
        assert torch.equal(state[-1].cpu(), stale[-1])


# ------------------------------------------------------------------------------------------------ small operations
@pytest.mark.parametrize("T", [5, 40])
@pytest.mark.parametrize("s,W", [(1, 300), (2, 300), (3, 1100), (8, 300), (4, 3000), (8, 3000), (3, 5000), (2, 9000)])
def test_streams_step(s, W, T):
    """Narrow rows live in registers (by stream count, width and row count), wide ones go column block by column
    block."""
    from lit_gpt import seq_ops

    dev = torch.device("cuda", 0)
    g = torch.Generator().manual_seed(s)
    x = torch.randn(T, s, W, generator=g)
    y, mix, out, read = torch.randn(T, W, generator=g), torch.randn(s, s, generator=g), torch.randn(s, generator=g), \
        torch.randn(s, generator=g)
    nw = torch.randn(W, generator=g)
    nx = torch.einsum("ij,tiw->tjw", mix.double(), x.double()) + out.double()[None, :, None] * y.double()[:, None, :]
    u = torch.einsum("j,tjw->tw", read.double(), nx)
    xd = x.to(dev)
    h, h16 = seq_ops.streams_step(xd, y=y.to(dev), mix=mix.to(dev), out=out.to(dev), read=read.to(dev),
                                  norm_w=nw.to(dev), eps=1e-5, bf16_copy=True)
    assert (xd.cpu().double() - nx).abs().max() < 1e-5
    assert (h.cpu().double() - orc.norm_plain(u, nw.double(), 1e-5)).abs().max() < 1e-4
    assert torch.equal(h16.cpu(), h.cpu().bfloat16())
    plain = seq_ops.streams_step(xd, read=read.to(dev))  # the weighted sum alone, nothing written
    assert (plain.cpu().double() - u).abs().max() < 1e-5 and (xd.cpu().double() - nx).abs().max() < 1e-5


def test_clamped_unit():
    from lit_gpt import seq_ops

    dev = torch.device("cuda", 0)
    z = torch.linspace(-6, 6, 2 * 77).reshape(2, 77).repeat(3, 1).contiguous()
    a, b = z[:, :40], z.flip(1)[:, :40]
    got = seq_ops.glu_clamped(z.to(dev), 0, 37, 40, alpha=1.702, limit=2.5, shift=1.0)
    gg, uu = a.clamp(max=2.5), z[:, 37:77].clamp(-2.5, 2.5)
    assert (got.cpu() - gg * torch.sigmoid(1.702 * gg) * (uu + 1.0)).abs().max() < 1e-5


# ------------------------------------------------------------------------------------------------ entry points
def follows_plain_greedy(cfg, w, prompt, out):
    """Every continued token is the plain implementation's argmax wherever that has a clear margin."""
    lg = orc.forward(cfg, w, out[:-1])
    clear = [i for i in range(len(prompt) - 1, len(out) - 1) if float(torch.topk(lg[i], 2).values.diff().abs()) > 1e-3]
    return bool(clear) and all(out[i + 1] == int(lg[i].argmax()) for i in clear)


def test_greedy_generation_through_the_entry_points():
    from generate.base import generate
    from generate.batch import BatchEngine

    cfg = make_cfg(MIXED[:3], streams=2)
    model, w = build(cfg, seed=7)
    prompts = [tokens_of(9, cfg["vocab"], seed=1), tokens_of(4, cfg["vocab"], seed=2), tokens_of(15, cfg["vocab"], seed=3)]
    new = 8
    eng = BatchEngine(model, max_seq_length=24)
    batched = eng.generate(prompts, new)
    assert not eng.live
    for p, out in zip(prompts, batched):
        assert out[:len(p)] == p and len(out) == len(p) + new
        assert follows_plain_greedy(cfg, w, p, out)
    assert BatchEngine(model, max_seq_length=24).generate(prompts, new, use_graph=True) == batched
    model.set_kv_cache(1, 24)
    single = generate(model, torch.tensor(prompts[0], dtype=torch.int32, device="cuda"), len(prompts[0]) + new,
                      temperature=0.0).cpu().tolist()
    assert single == batched[0]
    sampled = BatchEngine(model, max_seq_length=24).generate(prompts, 3, temperature=0.8, top_k=5)
    assert [len(o) for o in sampled] == [len(p) + 3 for p in prompts]


def test_command_line_serves_a_checkpoint_folder(tmp_path, capsys):
    import json

    from safetensors.torch import save_file

    from generate.base import main
    from lit_gpt.config import LayeredConfig
    from lit_gpt.layered import LayeredGPT

    cfg = make_cfg(MIXED[:3], vocab=70, streams=2)
    w = LayeredGPT.random_weights(LayeredConfig.from_dict(cfg), seed=15)
    save_file({k: v.contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    main(checkpoint_dir=tmp_path, max_new_tokens=5, temperature=0.0, top_k=None, prompt_len=7, precision="32-true")
    ids = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert len(ids) == 12
    assert follows_plain_greedy(cfg, w, ids[:7], ids)


def test_checkpoint_folder_through_registry_and_runner(tmp_path):
    import json
    import subprocess
    import sys

    import numpy as np
    from safetensors.torch import save_file

    from lit_gpt.config import LayeredConfig, load_config, model_class
    from lit_gpt.layered import LayeredGPT

    REPO = Path(__file__).resolve().parent.parent
    cfg = make_cfg(MIXED, streams=3)
    weights = LayeredGPT.random_weights(LayeredConfig.from_dict(cfg), seed=11)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in weights.items()}, str(tmp_path / "model.safetensors"))
    config = load_config(tmp_path)
    assert model_class(config) is LayeredGPT
    a, b = tokens_of(14, cfg["vocab"], seed=1), tokens_of(6, cfg["vocab"], seed=2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:10], "want": [3, 9]}, {"id": "b", "tokens": b[:5], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[10:11], "want": [0]}, {"id": "b", "tokens": b[5:], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[11:12], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[12:], "want": [1]}], "end": ["a"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(tmp_path), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "32"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.split("\n") if l.startswith("done")] == [f"done {i}" for i in range(4)]
    wa, wb = orc.forward(cfg, weights, a), orc.forward(cfg, weights, b)
    V = cfg["vocab"]
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    got1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, V))
    got3 = torch.from_numpy(np.fromfile(out / "3.f32", dtype="<f4").reshape(-1, V))
    assert not (out / "2.f32").exists()
    assert rel_err(got0, wa[[3, 9]]).max() < TOL32
    assert rel_err(got1, torch.stack([wa[10], wb[5]])).max() < TOL32
    assert rel_err(got3, wa[13:14]).max() < TOL32

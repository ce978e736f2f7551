"""The layered models (retention / latent-attention mixers, gated and sparse feed-forwards, per-layer token input,
layer loops) on the GPU against the plain CPU implementation in oracle/bavesun.py.

Every test makes its own small configuration and random weights. fp32 weights are compared tightly (the kernels then
run plain fp32); bf16 weights within the noise of bf16 operands. Schedules (whole prompt, token by token, portions,
batches, reused slots) must not change a position's logits beyond rounding.
"""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import bavesun as ob  # noqa: E402


# ------------------------------------------------------------------------------------------------ configurations
def ret(heads=2, dim=16, vdim=16, rot_dims=None, base=10000.0, decay=None):
    decay = decay or [1.0 - 2.0 ** -(3 + i) for i in range(heads)]
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay,
                                           "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base}}}


def lat(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=24, base=5000.0, scale=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
                      "rot": {"dims": rot_dim, "base": base},
                      "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(ff=24, experts=5, top=2):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_cfg(layers, width=48, vocab=61, loop=None, side=6, eps=1e-5, emb_scale=5.0):
    cfg = {"architecture": "Bavesun", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": emb_scale}, "layers": [dict(l[0], mlp=l[1]) for l in layers]}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


MIXED = [(ret(), dense()), (lat(), moe()), (ret(heads=3, dim=8, vdim=12, rot_dims=4), moe(top=1)), (lat(heads=3, kv_rank=64), None)]


def build(cfg, dtype=torch.float32, seed=0):
    from lit_gpt.config import LayeredConfig
    from lit_gpt.layered import LayeredGPT

    config = LayeredConfig.from_dict(cfg)
    weights = LayeredGPT.random_weights(config, seed=seed)
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
    return (d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9))


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


def oracle_logits(cfg, weights, toks):
    return ob.forward(cfg, weights, toks)


TOL32, TOL16 = 2e-4, 6e-2


# ------------------------------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("layers,side", [
    ([(ret(), None)], 0),
    ([(ret(heads=1, dim=24, vdim=8, rot_dims=6, decay=[1.0]), None)], 0),
    ([(ret(heads=2, dim=72, vdim=80), None)], 0),
    ([(lat(), None)], 0),
    ([(lat(heads=1, dim=4, rot_dim=2, vdim=6, kv_rank=10), None)], 0),
    ([(lat(heads=3, dim=16, rot_dim=72, vdim=8, kv_rank=136), None)], 0),
    ([(lat(heads=2, dim=8, rot_dim=6, vdim=8, kv_rank=64), None)], 0),
    ([(lat(heads=2, dim=8, rot_dim=72, vdim=8, kv_rank=128), None)], 0),
    ([(lat(heads=1, dim=8, rot_dim=4, vdim=8, kv_rank=640), None)], 0),
    ([(ret(heads=1, dim=272, vdim=16, rot_dims=20), None)], 0),
    ([(lat(heads=2, dim=8, rot_dim=16, vdim=24, kv_rank=192), dense())], 0),
    ([(ret(), dense())], 0),
    ([(ret(), moe())], 0),
    ([(lat(), moe(ff=7, experts=1, top=1))], 0),
    ([(lat(), moe(ff=10, experts=70, top=5))], 0),
    ([(ret(), None)], 6),
    ([(lat(), dense(ff=9))], 1),
])
def test_single_layer_against_oracle(layers, side):
    cfg = make_cfg(layers, side=side)
    model, w = build(cfg)
    toks = tokens_of(37, cfg["vocab"])
    got = engine_logits(model, [toks], [[len(toks)]])[0]
    assert rel_err(got, oracle_logits(cfg, w, toks)).max() < TOL32


@pytest.mark.parametrize("width,vocab", [(50, 33), (8, 5), (136, 300)])
def test_odd_sizes_and_loops(width, vocab):
    """Widths that are no multiple of the vector loads, a loop over all layers, one over a single layer, times = 1."""
    for loop in ((0, 4, 2), (1, 2, 3), (2, 4, 1), None):
        cfg = make_cfg(MIXED, width=width, vocab=vocab, loop=loop, side=3)
        model, w = build(cfg, seed=3)
        toks = tokens_of(21, vocab, seed=1)
        got = engine_logits(model, [toks], [[len(toks)]])[0]
        assert rel_err(got, oracle_logits(cfg, w, toks)).max() < TOL32, loop


def test_layer_residuals_against_oracle():
    """The residual stream after every layer run, loop passes included."""
    from lit_gpt import seq_ops
    from lit_gpt.mixers import StepBatch

    cfg = make_cfg(MIXED, loop=(0, 3, 2))
    model, w = build(cfg)
    toks = tokens_of(19, cfg["vocab"])
    want = []
    ob.forward(cfg, w, toks, want)
    model.set_kv_cache(1, 32)
    step = StepBatch.build([(0, 0, toks)], model.device)
    x = seq_ops.embed(step.tokens, model.embed, model.config.embedding_scale)
    assert len(model.runs) == len(want) == 7
    for run, layer in enumerate(model.runs):
        model.blocks[layer](x, step, model.caches[run])
        assert (x.cpu().double() - want[run]).abs().max() < 2e-4 * want[run].abs().max(), run


def test_bf16_weights_within_operand_noise():
    cfg = make_cfg(MIXED, loop=(0, 2, 2))
    model, w = build(cfg, dtype=torch.bfloat16)
    toks = tokens_of(150, cfg["vocab"])
    whole = engine_logits(model, [toks], [[len(toks)]])[0]
    e = rel_err(whole, oracle_logits(cfg, w, toks))
    assert e.median() < TOL16 / 3 and (e > TOL16).float().mean() < 0.05, (e.median(), e.max())
    # token by token through the streaming kernels: same operands, other summation order
    single = engine_logits(model, [toks], [[1] * len(toks)])[0]
    e2 = rel_err(single, whole)
    assert e2.median() < TOL16 / 3 and (e2 > TOL16).float().mean() < 0.05, (e2.median(), e2.max())


# ------------------------------------------------------------------------------------------------ schedules
def test_prefill_equals_token_by_token_and_portions():
    cfg = make_cfg(MIXED, loop=(1, 3, 2))
    model, w = build(cfg, seed=5)
    toks = tokens_of(45, cfg["vocab"], seed=2)
    want = oracle_logits(cfg, w, toks)
    for cuts in ([45], [1] * 45, [2] * 22 + [1], [3, 2, 17, 1, 1, 9, 12], [44, 1], [1, 44]):
        got = engine_logits(model, [toks], [cuts])[0]
        assert rel_err(got, want).max() < TOL32, cuts


def test_first_tokens_of_a_sequence():
    """A prompt of one token, then decoding: position 0 sees itself only (and the sink)."""
    cfg = make_cfg(MIXED)
    model, w = build(cfg, seed=6)
    toks = tokens_of(6, cfg["vocab"], seed=3)
    want = oracle_logits(cfg, w, toks)
    got = engine_logits(model, [toks], [[1] * 6], max_seq=8)[0]
    assert rel_err(got, want).max() < TOL32
    assert rel_err(engine_logits(model, [toks[:1]], [[1]])[0], want[:1]).max() < TOL32


def test_unequal_batch_equals_each_alone():
    cfg = make_cfg(MIXED, loop=(0, 2, 2))
    model, w = build(cfg, seed=7)
    seqs = [tokens_of(n, cfg["vocab"], seed=10 + n) for n in (33, 5, 58, 1 + 20)]
    # prompts of different lengths in one step, then decoded together; the shorter ones end earlier
    cuts = [[20] + [1] * 13, [2] + [1] * 3, [40] + [1] * 18, [1] + [1] * 20]
    got = engine_logits(model, seqs, cuts, max_seq=64)
    for s, g in zip(seqs, got):
        assert rel_err(g, oracle_logits(cfg, w, s)).max() < TOL32
    alone = [engine_logits(model, [s], [c], max_seq=64)[0] for s, c in zip(seqs, cuts)]
    for a, g in zip(alone, got):
        assert rel_err(g, a).max() < 1e-5


def test_slots_freed_and_used_again_and_grown():
    """Requests that end give their slot back; a later request in the same slot must not see what was there, and
    more live requests than the caches were built for make them grow without losing state."""
    from generate.batch import BatchEngine

    cfg = make_cfg(MIXED)
    model, w = build(cfg, seed=8)
    V = cfg["vocab"]
    eng = BatchEngine(model, max_seq_length=40, slots=1)
    a, b, c, d = (tokens_of(n, V, seed=20 + n) for n in (30, 12, 25, 9))
    la = eng.step([("a", a[:20], list(range(20)))])
    assert eng.live["a"][0] == 0
    lb = eng.step([("a", a[20:21], [0]), ("b", b[:1], [0])])  # b joins in a second slot: the caches grow
    assert eng.live["b"][0] == 1 and model.slots >= 2
    rest_a = eng.step([("a", a[21:], list(range(9)))], end=["a"])
    # c takes a's slot 0 (longer history than c's was there), d takes slot 2
    lc = eng.step([("c", c, list(range(25))), ("d", d, list(range(9)))], end=["d"])
    assert eng.live["c"][0] == 0 and eng.pool.size == 3
    rest_b = eng.step([("b", b[1:], list(range(11)))], end=["b", "c"])
    assert not eng.live and sorted(eng.pool.free) == [0, 1, 2]
    got_a = torch.cat([la, lb[:1], rest_a]).cpu()
    got_b = torch.cat([lb[1:], rest_b]).cpu()
    for got, toks in ((got_a, a), (got_b, b), (lc[:25].cpu(), c), (lc[25:].cpu(), d)):
        assert rel_err(got, oracle_logits(cfg, w, toks)).max() < TOL32


def test_long_decoding_keeps_state():
    """A slow decay (2^-11 per token) over 300 decoded tokens: the state is carried step by step in fp32."""
    layers = [(ret(heads=2, dim=8, vdim=8, decay=[1.0 - 2.0 ** -11, 0.9]), dense(16)), (lat(kv_rank=12), None)]
    cfg = make_cfg(layers, width=24, vocab=40, side=0)
    model, w = build(cfg, seed=9)
    toks = tokens_of(330, 40, seed=4)
    want = oracle_logits(cfg, w, toks)
    got = engine_logits(model, [toks], [[30] + [1] * 300])[0]
    assert rel_err(got, want).max() < 5e-4
    assert rel_err(engine_logits(model, [toks], [[330]])[0], want).max() < 5e-4


# ------------------------------------------------------------------------------------------------ crafted cases
def _plain_latent_attention(qc, qr, c, kr, sink, scale):
    """One head, query at the last position: softmax over all rows of [c | kr] with the sink in the denominator."""
    s = (c.double() @ qc.double() + kr.double() @ qr.double()) * scale
    m = max(float(s.max()), float(sink))
    e = torch.exp(s - m)
    return (e[:, None] * c.double()).sum(0) / (e.sum() + math.exp(float(sink) - m))


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
def test_far_key_and_sink_stand_out(cache_dtype):
    """Among 700 cached rows one far key (position 3) is aligned with the query and scaled so that its score stands
    out: the output must be that row, in a prompt step and in a decode step; a large sink must take its share."""
    from lit_gpt import seq_ops

    dev = torch.device("cuda", 0)
    g = torch.Generator().manual_seed(5)
    H, d, dr, r, S = 2, 4, 6, 64, 704
    n = 700
    c = 0.1 * torch.randn(n, r, generator=g)
    kr = torch.randn(n, dr, generator=g)
    qc = torch.randn(H, r, generator=g) * 0.1
    qr = torch.randn(H, dr, generator=g) * 0.1
    c[3] = 0.5 * torch.sign(torch.randn(r, generator=g))
    qc[0] = (160.0 / r) * c[3]  # head 0: score 40 at row 3, about +-1 elsewhere
    if cache_dtype == torch.bfloat16:
        c = c.to(torch.bfloat16).float()
    cache_c = torch.zeros(2, S, r, dtype=cache_dtype)
    cache_kr = torch.zeros(2, S, dr)
    cache_c[1, :n], cache_kr[1, :n] = c.to(cache_dtype), kr
    for sink in (torch.tensor([-30.0, 0.3]), torch.tensor([42.0, 3.0])):
        for T in (1, 5):  # a decode step, and the last rows of a prompt portion
            pos = torch.arange(n - T, n, dtype=torch.int32)
            proj = torch.zeros(T, H * (d + dr))
            proj.view(T, H, d + dr)[:, :, d:] = qr
            out = seq_ops.latent_attention(qc.reshape(1, -1).repeat(T, 1).contiguous().to(dev), proj.to(dev), 0,
                                           cache_c.to(dev), cache_kr.to(dev), sink.to(dev),
                                           torch.ones(T, dtype=torch.int32, device=dev), pos.to(dev), H=H, d=d, dr=dr,
                                           r=r, scale=1.0).cpu().view(T, H, r)
            if T > 1:  # the same rows through the prompt form (one sequence in slot 1 that starts at n - T)
                i32 = lambda *x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
                tiles = seq_ops.latent_attention_tiles(qc.reshape(1, -1).repeat(T, 1).contiguous().to(dev), proj.to(dev), 0,
                                                       cache_c.to(dev), cache_kr.to(dev), sink.to(dev), i32(0, T), i32(1),
                                                       i32(n - T), T, H=H, d=d, dr=dr, r=r, scale=1.0).cpu().view(T, H, r)
                assert (tiles - out).abs().max() < 1e-4 * max(1.0, float(out.abs().max()))
            for t in range(T):
                L = int(pos[t]) + 1
                for h in range(H):
                    want = _plain_latent_attention(qc[h], qr[h], c[:L], kr[:L], sink[h], 1.0)
                    assert (out[t, h].double() - want).abs().max() < 1e-4 * max(1.0, float(want.abs().max()))
            if float(sink[0]) < 0:
                assert (out[:, 0] - c[3]).abs().max() < 1e-3  # all the weight on the far key
            else:
                assert (out[:, 0] - c[3] * (1.0 / (1.0 + math.exp(2.0)))).abs().max() < 1e-2  # the sink's share


def _plain_retention(q, k, v, decay):
    """One head: S <- decay S + k v^T, o = S^T q, token after token. q, k (T, d), v (T, dv) -> (T, dv)."""
    S = torch.zeros(q.shape[1], v.shape[1], dtype=torch.float64)
    out = []
    for t in range(q.shape[0]):
        S = decay * S + torch.outer(k[t].double(), v[t].double())
        out.append(S.T @ q[t].double())
    return torch.stack(out)


def test_retention_far_token_survives():
    """decay 1 and a decay near 1: the key of token 5 is scaled so that it dominates the state along one direction;
    queries 500 positions later along that direction must return its value (times decay^distance), in one prompt
    step, with the state carried over portions, and in one-token steps, also in a slot that was used before."""
    from lit_gpt import seq_ops

    dev = torch.device("cuda", 0)
    g = torch.Generator().manual_seed(3)
    H, d, dv, T = 2, 8, 12, 520
    decay = [1.0, 1.0 - 2.0 ** -9]
    q = 0.1 * torch.randn(T, H, d, generator=g)
    k = 0.1 * torch.randn(T, H, d, generator=g)
    v = torch.randn(T, H, dv, generator=g)
    k[5, :, 0] = 50.0
    q[-20:, :, 0] = 1.0
    want = torch.stack([_plain_retention(q[:, h], k[:, h], v[:, h], decay[h]) for h in range(H)], 1)
    far = torch.stack([50.0 * v[5, h].double() * decay[h] ** (T - 1 - 5) for h in range(H)])
    assert (want[-1] - far).abs().max() < 0.2 * far.abs().max()  # the far token carries the answer
    ld = 2 * H * d + H * dv
    proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).contiguous().to(dev)
    dec = torch.tensor(decay, device=dev)
    for cuts, side_by_side in (([T], True), ([T], False), ([500] + [1] * 20, True), ([64] * 8 + [8], False),
                               ([200, 129, 191], True), ([2] * 260, False)):
        state = torch.full((3, H, d, dv), 7.0, device=dev)  # stale values of an earlier owner of the slot
        outs, at = [], 0
        for n in cuts:
            i32 = lambda *x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
            outs.append(seq_ops.retention(proj[at:at + n].contiguous(), 0, H * d, 2 * H * d, state, dec, None,
                                          i32(0, n), i32(2), i32(at), H=H, d=d, dv=dv, rot_dims=0, k_scale=1.0,
                                          max_len=n if side_by_side else 0,
                                          pos=torch.arange(at, at + n, dtype=torch.int32, device=dev)))
            at += n
        got = torch.cat(outs).cpu().view(T, H, dv).double()
        assert (got - want).abs().max() < 1e-4 * want.abs().max(), cuts
    assert ld == proj.shape[1]


def test_router_picks_and_weights():
    """Crafted router logits: the chosen experts, their order among equals and the softmax over the chosen only."""
    from lit_gpt import seq_ops

    z = torch.tensor([[0.0, 3.0, 1.0, 3.0, -1.0, 2.5], [5.0, -2.0, -2.0, 0.0, 0.0, 0.0]])
    pad = torch.cat([torch.full((2, 3), 99.0), z], 1).cuda().contiguous()  # logits start at column 3 of the row
    ids, wts = seq_ops.moe_route(pad, 3, 6, 3)
    assert ids.cpu().tolist() == [[1, 3, 5], [0, 3, 4]]
    want0 = torch.softmax(torch.tensor([3.0, 3.0, 2.5]), 0)
    want1 = torch.softmax(torch.tensor([5.0, 0.0, 0.0]), 0)
    assert torch.allclose(wts.cpu(), torch.stack([want0, want1]), atol=1e-6)
    ids1, wts1 = seq_ops.moe_route(pad, 3, 6, 1)
    assert ids1.cpu().tolist() == [[1], [0]] and torch.allclose(wts1.cpu(), torch.ones(2, 1))


# ------------------------------------------------------------------------------------------------ kernels
@pytest.mark.parametrize("M,N,K", [(1, 40, 64), (3, 33, 50), (8, 130, 136), (9, 24, 8), (70, 130, 200), (200, 300, 72),
                                   (130, 5, 30)])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_linear_kernels(M, N, K, wdtype):
    from lit_gpt import seq_ops

    g = torch.Generator().manual_seed(M * 1000 + N)
    a = torch.randn(M, K, generator=g)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    y0 = torch.randn(M, N, generator=g)
    aa = a.to(torch.bfloat16).double() if wdtype == torch.bfloat16 else a.double()
    want = aa @ w.double().T
    y = y0.clone().cuda()
    seq_ops.linear(a.cuda(), w.to(wdtype).cuda(), M=M, N=N, K=K, y=y, lda=K, ldy=N, accumulate=True)
    assert (y.cpu().double() - (y0.double() + want)).abs().max() < 1e-4 * K ** 0.5
    y = torch.empty(M, N).cuda()
    seq_ops.linear(a.cuda(), w.to(wdtype).cuda(), M=M, N=N, K=K, y=y, lda=K, ldy=N, act=seq_ops.ACT_RELU2)
    assert (y.cpu().double() - torch.relu(want) ** 2).abs().max() < 1e-4 * K


@pytest.mark.parametrize("T", [4, 150])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_linear_per_head_and_grouped(T, wdtype):
    from lit_gpt import seq_ops

    g = torch.Generator().manual_seed(T)
    H, d, extra, r = 3, 8, 4, 20
    a = torch.randn(T, 5 + H * (d + extra), generator=g)
    w = torch.randn(H, r, d, generator=g).to(torch.bfloat16)
    y = torch.zeros(T, H * r).cuda()
    seq_ops.linear(a.cuda(), w.to(wdtype).cuda(), M=T, N=r, K=d, y=y, a_off=5, lda=a.shape[1], ldy=H * r, batch=H,
                   stride_a=d + extra, stride_w=r * d, stride_y=r)
    src = a[:, 5:].reshape(T, H, d + extra)[:, :, :d]
    src = src.to(torch.bfloat16).double() if wdtype == torch.bfloat16 else src.double()
    want = torch.einsum("thd,hrd->thr", src, w.double()).reshape(T, H * r)
    assert (y.cpu().double() - want).abs().max() < 1e-4
    # grouped: rows sorted by expert, each range times its expert's matrix
    E, top, N, K = 4, 2, 12, 16
    ids = torch.randint(0, E, (T, top), generator=g).to(torch.int32)
    z_start, tok_of, where = seq_ops.moe_sort(ids.cuda(), E)
    flat = ids.reshape(-1)
    assert z_start.cpu().tolist() == [0] + torch.cumsum(torch.bincount(flat.long(), minlength=E), 0).tolist()
    wh = where.cpu().long()
    assert sorted(wh.tolist()) == list(range(T * top))  # a permutation ...
    assert tok_of.cpu()[wh].tolist() == [i // top for i in range(T * top)]  # ... that remembers every pair's token
    for e in range(E):  # ... and puts every pair into its expert's range
        assert all(int(z_start[e]) <= int(w) < int(z_start[e + 1]) for w in wh[flat == e])
    order = torch.empty(T * top, dtype=torch.long)
    order[wh] = torch.arange(T * top)
    hmat = torch.randn(T, K, generator=g)
    we = torch.randn(E, N, K, generator=g).to(torch.bfloat16)
    out = torch.zeros(T * top, N).cuda()
    seq_ops.linear(hmat.cuda(), we.to(wdtype).cuda(), M=T * top, N=N, K=K, y=out, lda=K, ldy=N, batch=E,
                   stride_w=N * K, a_rows=tok_of, z_start=z_start)
    hh = hmat.to(torch.bfloat16).double() if wdtype == torch.bfloat16 else hmat.double()
    want = torch.stack([hh[int(tok_of[i])] @ we[int(flat[order[i]])].double().T for i in range(T * top)])
    assert (out.cpu().double() - want).abs().max() < 1e-4


def test_sparse_forms_agree():
    """The streaming form (few pairs) and the grouped form (a prompt) of the experts give the same sums."""
    from lit_gpt.mixers import SparseFeedForward

    cfg = make_cfg([(ret(), moe(ff=20, experts=6, top=3))], side=0)
    model, _ = build(cfg, seed=12)
    ff = model.blocks[0].mlp
    T = 12
    g = torch.Generator().manual_seed(2)
    h = torch.randn(T, cfg["width"], generator=g).cuda()
    proj = torch.randn(T, model.blocks[0].w_in.shape[0], generator=g).cuda()
    outs = []
    for limit in (10 ** 6, 0):
        x = torch.zeros(T, cfg["width"]).cuda()
        SparseFeedForward.STREAM_PAIRS, keep = limit, SparseFeedForward.STREAM_PAIRS
        try:
            ff(proj, h, x)
        finally:
            SparseFeedForward.STREAM_PAIRS = keep
        outs.append(x.cpu())
    assert (outs[0] - outs[1]).abs().max() < 1e-5 * outs[0].abs().max()


# ------------------------------------------------------------------------------------------------ generation
def test_greedy_generation_through_entry_point_and_scheduler():
    """generate.base.generate (one sequence, the framework's sampler) and BatchEngine.generate (several prompts of
    unequal length) against greedy decoding on the oracle, wherever the oracle's margin is clear."""
    from generate.base import generate
    from generate.batch import BatchEngine

    cfg = make_cfg(MIXED, loop=(0, 2, 2))
    model, w = build(cfg, seed=13)
    V = cfg["vocab"]
    prompts = [tokens_of(n, V, seed=30 + n) for n in (9, 3, 17)]
    new = 12
    model.set_kv_cache(1, 40)
    single = generate(model, torch.tensor(prompts[0], dtype=torch.int32, device="cuda"), len(prompts[0]) + new,
                      temperature=0.0).cpu().tolist()
    eng = BatchEngine(model, max_seq_length=40)
    batched = eng.generate(prompts, new)
    assert batched[0] == single and not eng.live
    checked = 0
    for p, out in zip(prompts, batched):
        assert out[:len(p)] == p and len(out) == len(p) + new
        lg = oracle_logits(cfg, w, out[:-1])
        for i in range(len(p) - 1, len(out) - 1):
            top2 = torch.topk(lg[i], 2).values
            if float(top2[0] - top2[1]) > 1e-3:
                assert out[i + 1] == int(torch.argmax(lg[i]))
                checked += 1
    assert checked > 2 * new


def test_captured_decode_steps_equal_eager_steps():
    """The one-token steps as replays of one HIP graph: every replay must give the eager step's token and leave the
    caches and states as the eager step would, also after other eager work and a second capture in between."""
    from generate.batch import BatchEngine

    cfg = make_cfg(MIXED, loop=(0, 2, 2))
    model, _ = build(cfg, seed=16)
    V = cfg["vocab"]
    prompts = [tokens_of(n, V, seed=40 + n) for n in (11, 4, 23)]
    eng = BatchEngine(model, max_seq_length=48)
    eager = eng.generate(prompts, 14)
    for _ in range(2):
        assert eng.generate(prompts, 14, use_graph=True) == eager
        assert eng.generate(prompts[::-1], 3) == [e[:len(p) + 3] for e, p in zip(eager[::-1], prompts[::-1])]
    assert not eng.live
    # replay by replay against the logits of the eager steps
    ids = ["x", "y", "z"]
    logits = eng.step([(i, p, [len(p) - 1]) for i, p in zip(ids, prompts)])
    first = [int(torch.argmax(logits[i])) for i in range(3)]
    graph = eng.decode_graph(ids, first)
    for n in range(6):
        drawn = graph.step().cpu().tolist()
        assert drawn == [e[len(p) + 1 + n] for e, p in zip(eager, prompts)], n
        torch.cuda.synchronize()
    eng.step([], end=ids)


def test_checkpoint_folder_round_trip(tmp_path):
    """config.json + model.safetensors written to a folder: the registry picks the class, the loader the tensors."""
    import json
    import struct

    from lit_gpt.config import LayeredConfig, load_config, model_class

    cfg = make_cfg(MIXED[:2])
    config = LayeredConfig.from_dict(cfg)
    cls = model_class(config)
    w = cls.random_weights(config, seed=14)
    header, blob = {}, b""
    for name, t in w.items():
        raw = t.contiguous().view(torch.uint8).numpy().tobytes()
        header[name] = {"dtype": "BF16", "shape": list(t.shape), "data_offsets": [len(blob), len(blob) + len(raw)]}
        blob += raw
    hj = json.dumps(header).encode()
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", len(hj)) + hj + blob)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    assert isinstance(load_config(tmp_path), LayeredConfig)
    model = cls.from_checkpoint(tmp_path, device=torch.device("cuda", 0), dtype=torch.float32)
    toks = tokens_of(11, cfg["vocab"])
    got = engine_logits(model, [toks], [[11]])[0]
    assert rel_err(got, oracle_logits(cfg, w, toks)).max() < TOL32


def test_command_line_serves_a_checkpoint_folder(tmp_path, capsys):
    """generate/base.py's main on a folder with config.json + model.safetensors of a registered architecture."""
    import json
    import struct

    from generate.base import main
    from lit_gpt.config import LayeredConfig
    from lit_gpt.layered import LayeredGPT

    cfg = make_cfg(MIXED[:2], vocab=70)
    w = LayeredGPT.random_weights(LayeredConfig.from_dict(cfg), seed=15)
    header, blob = {}, b""
    for name, t in w.items():
        raw = t.contiguous().view(torch.uint8).numpy().tobytes()
        header[name] = {"dtype": "BF16", "shape": list(t.shape), "data_offsets": [len(blob), len(blob) + len(raw)]}
        blob += raw
    hj = json.dumps(header).encode()
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", len(hj)) + hj + blob)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    main(checkpoint_dir=tmp_path, max_new_tokens=5, temperature=0.0, top_k=None, prompt_len=7, precision="32-true")
    ids = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert len(ids) == 12
    g = torch.Generator(device="cpu").manual_seed(1234)
    prompt = torch.randint(0, 70, (7,), generator=g, dtype=torch.int32).tolist()
    assert ids[:7] == prompt
    lg = oracle_logits(cfg, w, ids[:-1])
    agree = [ids[i + 1] == int(torch.argmax(lg[i])) for i in range(6, 11)
             if float(torch.topk(lg[i], 2).values.diff().abs()) > 1e-3]
    assert agree and all(agree)

"""GPU tests of the mixer family (libexl3_mix.so, modules.py, vofanex.py, state_cache.py, generator.py) against the float64 oracle of
tests/mixer_oracle.py: every mechanism alone, whole models of several small shapes, prefill against token-by-token decoding, unequal
batches against each request alone, slots that are freed and used again, window and ring edges, sinks, far keys in the recurrent
state, long decoding, and greedy generation through the scheduler.  float32 runs are held to float32 rounding; bfloat16 runs to a
loose bar (the oracle does not round)."""
import math
import pytest
import torch
import mixer_oracle as mo

pytestmark = pytest.mark.gpu
F64 = torch.float64


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from exllamav3_amd import _lib
    _lib.mixlib()
    torch.backends.cuda.matmul.allow_tf32 = False
    return torch.device("cuda:0")


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).abs().max() / (b.abs().max() + 1e-30))


def batch_tensors(gpu, lens, pos0=None, slots=None):
    """cu, tok_seq, tok_pos, slots, pos0, len_after as int32 device tensors."""
    pos0 = pos0 or [0] * len(lens)
    slots = slots or list(range(len(lens)))
    cu = [0]
    for l in lens: cu.append(cu[-1] + l)
    seq = [i for i, l in enumerate(lens) for _ in range(l)]
    pos = [pos0[i] + j for i, l in enumerate(lens) for j in range(l)]
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=gpu)
    return mk(cu), mk(seq), mk(pos), mk(slots), mk(pos0), mk([p + l for p, l in zip(pos0, lens)])


TOL = {torch.float32: 2e-5, torch.bfloat16: 3e-2}


# ---- mechanisms alone -------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,W,lens", [(4, 2, 16, 24, 5, [17, 1, 9]), (3, 3, 40, 72, 64, [70]), (2, 1, 8, 8, 1, [6, 3]), (6, 2, 32, 130, 7, [20]), (2, 1, 96, 96, 37, [150, 66]), (1, 1, 136, 64, 100, [131]), (3, 1, 20, 12, 9, [40, 33]), (2, 1, 64, 64, 90, [300, 40]), (4, 2, 128, 128, 200, [530])])
def test_attention_prefill_then_decode_matches_oracle(gpu, dtype, H, G, d, dv, W, lens):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(H * 100 + W)
    extra = 2 * W + 3                                       # decoded tokens: the ring wraps more than once
    tot = [l + extra for l in lens]
    rnd = lambda *s: torch.randn(*s, generator=g).to(dtype)
    Q = [rnd(t, H, d) for t in tot]; K = [rnd(t, G, d) for t in tot]; V = [rnd(t, G, dv) for t in tot]; GT = [rnd(t, H) for t in tot]
    sink = torch.randn(H, generator=g)
    scale = 0.3
    ref = [mo.sliding_sink_attention(q.to(F64), k.to(F64), v.to(F64), scale, W, sink.to(F64), gt.to(F64), 1e-5) for q, k, v, gt in zip(Q, K, V, GT)]
    B, n_slots = len(lens), len(lens) + 2
    slots = [n_slots - 1 - i for i in range(B)]
    ring_k = torch.full((n_slots, W, G, d), float("nan"), dtype=dtype, device=gpu)       # stale / unwritten entries must never be read
    ring_v = torch.full((n_slots, W, G, dv), float("nan"), dtype=dtype, device=gpu)
    # prompt step
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens, slots=slots)
    cat = lambda xs, ls: torch.cat([x[:l] for x, l in zip(xs, ls)]).to(gpu)
    q, k, v, gt = cat(Q, lens).flatten(1), cat(K, lens).flatten(1), cat(V, lens).flatten(1), cat(GT, lens)
    n = sum(lens)
    vn = torch.empty((n, G, dv), dtype=dtype, device=gpu)
    mix_ops.attn_store(vn, ring_k, ring_v, k, v, seq, pos, sl, la, 1e-5)
    out = torch.empty((n, H * dv), dtype=dtype, device=gpu)
    want = torch.cat([r[:l] for r, l in zip(ref, lens)]).flatten(1)
    for mfma in ([False, True] if dtype == torch.bfloat16 else [False]):           # the lane-per-key kernel and the matrix-core kernel
        out.fill_(float("nan"))
        mix_ops.attn_prefill(out, q, k, vn, gt, sink.to(gpu), cu, seq, pos, H, scale, W, max_rows=max(lens), mfma=mfma)
        assert rel(out, want) < TOL[dtype], f"mfma={mfma}"
    # decode steps, all sequences together
    for s in range(extra):
        cur = [l + s for l in lens]
        cu, seq, pos, sl, p0, la = batch_tensors(gpu, [1] * B, pos0=cur, slots=slots)
        row = lambda xs: torch.stack([x[c] for x, c in zip(xs, cur)]).to(gpu)
        q, k, v, gt = row(Q).flatten(1), row(K).flatten(1), row(V).flatten(1), row(GT)
        vn = torch.empty((B, G, dv), dtype=dtype, device=gpu)
        mix_ops.attn_store(vn, ring_k, ring_v, k, v, seq, pos, sl, la, 1e-5)
        out = torch.empty((B, H * dv), dtype=dtype, device=gpu)
        mix_ops.attn_decode(out, q, ring_k, ring_v, gt, sink.to(gpu), sl, la, H, scale)
        want = torch.stack([r[c] for r, c in zip(ref, cur)]).flatten(1)
        assert rel(out, want) < TOL[dtype], f"decode step {s}"


@pytest.mark.parametrize("dtype,mfma", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
def test_attention_window_edge_and_sink_show_in_the_output(gpu, dtype, mfma):
    """One key is made to dominate (its score is far above all others): just inside the window the output is that key's value, just outside it is not;
    a huge sink takes the whole softmax mass and the output vanishes.  Both prefill kernels and the decode kernel; the edge lies inside a key tile
    of the matrix-core kernel for one row and on a tile border for another."""
    from exllamav3_amd import mix_ops
    d = dv = 16; T = 140
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    g = torch.Generator().manual_seed(3)
    for W, i in ((12, T - 1), (76, T - 1), (64, 127)):                # row 139, window 76: first visible key 64 = a tile border; row 127, window 64: the same
        q = (torch.randn(T, 1, d, generator=g) * 0.1).to(dtype); k = (torch.randn(T, 1, d, generator=g) * 0.1).to(dtype); v = torch.randn(T, 1, dv, generator=g).to(dtype)
        for j, inside in ((i - W + 1, True), (i - W, False)):
            kk = k.clone(); kk[j, 0] = (q[i, 0].float() / q[i, 0].float().norm() ** 2 * 60.0).to(dtype)            # score 60 against scores ~0.01
            cu, seq, pos, sl, p0, la = batch_tensors(gpu, [i + 1])
            ring_k = torch.zeros((1, W, 1, d), dtype=dtype, device=gpu); ring_v = torch.zeros((1, W, 1, dv), dtype=dtype, device=gpu)
            n = i + 1
            vn = torch.empty((n, 1, dv), dtype=dtype, device=gpu)
            mix_ops.attn_store(vn, ring_k, ring_v, kk[:n].flatten(1).to(gpu), v[:n].flatten(1).to(gpu), seq, pos, sl, la, 1e-5)
            out = torch.empty((n, dv), dtype=dtype, device=gpu)
            for sink, expect_zero in ((torch.full((1,), -30.0), False), (torch.full((1,), 200.0), True)):
                mix_ops.attn_prefill(out, q[:n].flatten(1).to(gpu), kk[:n].flatten(1).to(gpu), vn, None, sink.to(gpu), cu, seq, pos, 1, 1.0, W, max_rows=n, mfma=mfma)
                o = out[i].float().cpu()
                if expect_zero:
                    assert o.abs().max() < 1e-6
                else:
                    assert bool((o - vn[j, 0].float().cpu()).abs().max() < tol) == inside, (W, i, j)
                # the same row decoded against the ring (which holds the last W positions)
                mix_ops.attn_decode(out[:1], q[i].flatten().unsqueeze(0).to(gpu), ring_k, ring_v, None, sink.to(gpu), sl, la, 1, 1.0)
                o = out[0].float().cpu()
                if expect_zero:
                    assert o.abs().max() < 1e-6
                else:
                    assert bool((o - vn[j, 0].float().cpu()).abs().max() < tol) == inside, (W, i, j, "decode")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,dv,tau,rank,lens", [(2, 16, 32, 4.0, 4, [37, 1, 130]), (1, 48, 70, 16.0, 8, [200]), (3, 130, 64, 1.0, 3, [19, 66]), (2, 8, 8, 2.0, 1, [5])])
def test_gla_scan_whole_and_segmented_match_oracle_and_carry_state(gpu, dtype, H, d, dv, tau, rank, lens):
    from exllamav3_amd import mix_ops, _lib
    g = torch.Generator().manual_seed(H * 7 + d)
    rnd = lambda *s: torch.randn(*s, generator=g).to(dtype)
    B = len(lens)
    extra = 5
    tot = [l + extra for l in lens]
    Q = [rnd(t, H * d) for t in tot]; K = [rnd(t, H * d) * 0.5 for t in tot]; V = [rnd(t, H * dv) for t in tot]; LR = [rnd(t, rank) for t in tot]
    a2 = (torch.randn(H * d, rank, generator=g) * 1.5).to(dtype); a2b = torch.randn(H * d, generator=g) + 1.0
    qs = d ** -0.5
    refs = []
    for q, k, v, lr in zip(Q, K, V, LR):
        z = (lr.to(F64) @ a2.to(F64).T + a2b.to(F64)).view(-1, H, d)
        refs.append(mo.gla_recurrent(q.to(F64).view(-1, H, d) * qs, k.to(F64).view(-1, H, d), v.to(F64).view(-1, H, dv), z, tau)[0])
    mx = max(lens)
    for segments in [None] + [(-(-mx // L), L) for L in (16, 48, 112)]:
        slots = [B + 1 - i for i in range(B)]
        state = torch.full((B + 2, H, d, dv), float("nan"), dtype=torch.float32, device=gpu)      # a new sequence must not read its slot
        cu, seq, pos, sl, p0, la = batch_tensors(gpu, lens, slots=slots)
        cat = lambda xs: torch.cat([x[:l] for x, l in zip(xs, lens)]).to(gpu)
        o = torch.empty((sum(lens), H, dv), dtype=torch.float32, device=gpu)
        mix_ops.gla_scan(o, state, cat(Q), cat(K), cat(V), cat(LR), a2.to(gpu), a2b.to(gpu), cu, sl, p0, tau, qs, segments=segments)
        want = torch.cat([r[:l] for r, l in zip(refs, lens)])
        assert rel(o, want) < TOL[dtype], f"segments={segments}"
        for s in range(extra):                                                                   # decode from the carried state
            cur = [l + s for l in lens]
            cu, seq, pos, sl, p0, la = batch_tensors(gpu, [1] * B, pos0=cur, slots=slots)
            row = lambda xs: torch.stack([x[c] for x, c in zip(xs, cur)]).to(gpu)
            o = torch.empty((B, H, dv), dtype=torch.float32, device=gpu)
            mix_ops.gla_scan(o, state, row(Q), row(K), row(V), row(LR), a2.to(gpu), a2b.to(gpu), cu, sl, p0, tau, qs)
            want = torch.stack([r[c] for r, c in zip(refs, cur)])
            assert rel(o, want) < TOL[dtype], f"segments={segments} decode {s}"


def test_gla_keeps_a_far_key_and_forgets_with_the_decay(gpu):
    """With decays close to 1 a key written 300 tokens back still answers its query; with small decays it is gone.  The far key is the only one aligned with
    the last query, so a lost or misplaced state shows."""
    from exllamav3_amd import mix_ops, _lib
    H, d, dv, T, rank = 1, 16, 16, 320, 1
    g = torch.Generator().manual_seed(5)
    k = torch.randn(T, d, generator=g) * 0.05; q = torch.randn(T, d, generator=g) * 0.05; v = torch.randn(T, dv, generator=g)
    e = torch.zeros(d); e[3] = 1.0
    k[10] = e * 4.0; q[T - 1] = e * 4.0
    lr = torch.ones(T, rank); a2 = torch.zeros(d, rank)
    for bias, kept in ((12.0, True), (-2.0, False)):
        a2b = torch.full((d,), bias)
        ref = mo.gla_recurrent(q.to(F64).view(T, 1, d), k.to(F64).view(T, 1, d), v.to(F64).view(T, 1, dv), a2b.to(F64).expand(T, 1, d), 2.0)[0]
        for segments in (None, (4, 80), (20, 16)):
            cu, seq, pos, sl, p0, la = batch_tensors(gpu, [T])
            state = torch.zeros((1, 1, d, dv), device=gpu); o = torch.empty((T, 1, dv), device=gpu)
            mix_ops.gla_scan(o, state, q.to(gpu), k.to(gpu), v.to(gpu), lr.to(gpu), a2.to(gpu), a2b.to(gpu), cu, sl, p0, 2.0, 1.0, segments=segments)
            assert rel(o, ref) < 2e-5
            cos = torch.nn.functional.cosine_similarity(o[T - 1, 0].cpu(), v[10], dim=0)
            assert (cos > 0.95) == kept


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_row_kernels_match_oracle(gpu, dtype):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(1)
    n, width, ff, vocab = 7, 200, 330, 50
    table = torch.randn(vocab, width, generator=g).to(dtype); tokens = torch.randint(0, vocab, (n,), generator=g, dtype=torch.int32)
    nw = (1 + 0.1 * torch.randn(width, generator=g)); x = torch.empty((n, width), device=gpu); h = torch.empty((n, width), dtype=dtype, device=gpu)
    mix_ops.embed(x, h, table.to(gpu), tokens.to(gpu), 0.37, nw.to(gpu), 1e-5)
    xr = table.to(F64)[tokens.long()] * 0.37
    assert rel(x, xr) < 1e-6 and rel(h, mo.rms_norm(xr, nw.to(F64), 1e-5)) < TOL[dtype]
    y = torch.randn(n, width + 9, generator=g).to(dtype); r = torch.randn(n, width + 5, generator=g).to(dtype)
    x0 = x.clone().cpu().to(F64)
    mix_ops.gated_residual(x, y.to(gpu)[:, 9:], r.to(gpu)[:, :width], nw.to(gpu), h, 1e-5)
    xr = x0 + y.to(F64)[:, 9:] * torch.sigmoid(r.to(F64)[:, :width])
    assert rel(x, xr) < 1e-6 and rel(h, mo.rms_norm(xr, nw.to(F64), 1e-5)) < TOL[dtype]
    rows = torch.tensor([5, 0, 5], dtype=torch.int32); hw = torch.empty((3, width), dtype=dtype, device=gpu)
    mix_ops.rms_norm_rows(hw, x, rows.to(gpu), nw.to(gpu), 1e-5)
    assert rel(hw, mo.rms_norm(xr[rows.long()], nw.to(F64), 1e-5)) < TOL[dtype]
    z = torch.randn(n, ff + 3, generator=g).to(dtype) * 1.7; coef = torch.tensor([0.5, -0.25, 0.125, 0.3]); a = torch.empty((n, ff), dtype=dtype, device=gpu)
    mix_ops.polynorm(a, z.to(gpu)[:, 3:], coef.to(gpu), 1e-5)
    assert rel(a, mo.polynorm(z.to(F64)[:, 3:], coef, 1e-5)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,E,top,ff,width", [(5, 6, 2, 40, 72), (70, 4, 1, 32, 64), (3, 3, 3, 20, 40), (150, 8, 3, 96, 128), (21, 8, 2, 64, 136), (40, 3, 2, 24, 48)])
def test_router_and_experts_match_oracle(gpu, dtype, n, E, top, ff, width):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(n + E)
    logits = torch.randn(n, E, generator=g) * 2
    idx = torch.empty((n, top), dtype=torch.int32, device=gpu); wts = torch.empty((n, top), device=gpu)
    mix_ops.topk_softmax(idx, wts, logits.to(gpu))
    ti, tw = mo.route(logits.to(F64), top)
    assert torch.equal(idx.cpu().long(), ti) and rel(wts, tw) < 1e-6
    h = torch.randn(n, width, generator=g).to(dtype)
    wg = (torch.randn(E, ff, width, generator=g) / math.sqrt(width)).to(dtype); wu = (torch.randn(E, ff, width, generator=g) / math.sqrt(width)).to(dtype)
    wd = (torch.randn(E, width, ff, generator=g) / math.sqrt(ff)).to(dtype)
    ref = torch.zeros(n, width, dtype=F64)
    for t in range(n):
        for r in range(top):
            e = int(ti[t, r])
            ref[t] += tw[t, r] * ((mo.silu(h[t].to(F64) @ wg[e].to(F64).T) * (h[t].to(F64) @ wu[e].to(F64).T)) @ wd[e].to(F64).T)
    y = torch.empty((n, width), dtype=dtype, device=gpu); hid = torch.empty((n * top, ff), dtype=dtype, device=gpu)
    mix_ops.moe_gate_up(hid, h.to(gpu), wg.to(gpu), wu.to(gpu), idx)
    mix_ops.moe_down(y, hid, wd.to(gpu), idx, wts)
    assert rel(y, ref) < TOL[dtype]
    if mix_ops.moe_vector_layout(h, ff):
        y3 = torch.full_like(y, float("nan"))
        mix_ops.moe_expert_major(y3, h.to(gpu), wg.to(gpu), wu.to(gpu), wd.to(gpu), idx, wts)
        assert rel(y3, ref) < TOL[dtype]
    if True:
        y2 = torch.empty_like(y)
        mix_ops.moe_grouped(y2, h.to(gpu), wg.to(gpu), wu.to(gpu), wd.to(gpu), idx, wts)
        assert rel(y2, ref) < TOL[dtype]


# ---- whole models ---------------------------------------------------------------------------------------------------------------

SHAPES = {
    # attention first, no feed-forward in one layer, kv_heads == heads, vdim != dim, top 1
    "a": dict(vocab=80, width=48, layers=[dict(type="attention", heads=2, kv_heads=2, dim=24, vdim=40, window=6, mlp=("moe", 24, 3, 1)),
                                          dict(type="gla", heads=3, dim=20, vdim=12, tau=3.0, rank=2, mlp=None),
                                          dict(type="attention", heads=6, kv_heads=3, dim=8, vdim=8, window=33, mlp=("dense", 100))]),
    # recurrent layers only + a wide head dim, every expert chosen
    "b": dict(vocab=130, width=96, layers=[dict(type="gla", heads=1, dim=136, vdim=72, tau=8.0, rank=5, mlp=("moe", 40, 2, 2)),
                                           dict(type="gla", heads=2, dim=32, vdim=64, tau=1.5, rank=3, mlp=("dense", 64))]),
    # a window of one token and a window longer than every prompt
    "c": dict(vocab=64, width=64, layers=[dict(type="attention", heads=4, kv_heads=1, dim=16, vdim=16, window=1, mlp=("dense", 72)),
                                          dict(type="attention", heads=2, kv_heads=1, dim=32, vdim=20, window=500, mlp=("moe", 16, 5, 2)),
                                          dict(type="gla", heads=2, dim=16, vdim=16, tau=16.0, rank=4, mlp=("moe", 16, 4, 3))]),
}


@pytest.fixture(scope="module")
def models(gpu, tmp_path_factory):
    from exllamav3_amd.registry import load_model
    out = {}
    for name, s in SHAPES.items():
        cfg, t = mo.random_model(s["layers"], vocab=s["vocab"], width=s["width"], seed=len(name) + ord(name))
        d = str(tmp_path_factory.mktemp("m_" + name))
        mo.save_model(d, cfg, t)
        out[name] = (mo.OracleModel(cfg, t), {dt: load_model(d, gpu, dt) for dt in (torch.float32, torch.bfloat16)}, s["vocab"])
    return out


def toks(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def logit_err(got, ref, quantile=1.0):
    """Worst position's error (mean taken off, RMS over the vocabulary, relative to the spread of the logits).  bfloat16 runs pass quantile 0.5 (the median position): a router
    whose two best logits lie within bfloat16 rounding of the input may pick the other expert at one position, and the sequence state carries that on; the float32 run is held at every position."""
    got, ref = got.double().cpu(), ref.double()
    d = (got - ref); d = d - d.mean(-1, keepdim=True)
    e = (d.pow(2).mean(-1).sqrt() / ref.std(-1)).sort().values
    return float(e[min(len(e) - 1, int(quantile * len(e)))]) if quantile < 1.0 else float(e[-1])


QUANT = {torch.float32: 1.0, torch.bfloat16: 0.5}


@pytest.mark.parametrize("name", list(SHAPES))
def test_whole_prompt_and_every_layer_match_oracle(models, name):
    orc, ms, vocab = models[name]
    t = toks(vocab, 45, 1)
    taps = []
    ref = orc.forward(t, taps)
    for dt, bar in ((torch.float32, 3e-5), (torch.bfloat16, 6e-2)):
        m = ms[dt]; cache = m.new_cache(1); slot = cache.alloc()
        m.layer_taps = []
        got = m.step(cache.begin_step([(slot, t)], [list(range(len(t)))]), cache)
        if dt == torch.float32:
            for i, (a, b) in enumerate(zip(m.layer_taps, taps)):
                assert rel(a, b) < bar, f"layer {i} {dt}"
        m.layer_taps = None
        assert logit_err(got, ref, QUANT[dt]) < bar


@pytest.mark.parametrize("name", list(SHAPES))
def test_decoding_batches_and_slot_reuse_do_not_change_logits(models, name):
    """Three requests of unequal length: prompt step together, decoded together (the ring wraps, one request ends early and its slot is taken by a newcomer
    whose logits must equal its own fresh run), against the oracle's whole-sequence logits."""
    orc, ms, vocab = models[name]
    seqs = [toks(vocab, n, 10 + n) for n in (50, 9, 31)]
    cuts = [12, 1, 20]                                       # prompt lengths; the rest is decoded
    late = toks(vocab, 26, 99)
    refs = [orc.forward(s) for s in seqs]; ref_late = orc.forward(late)
    for dt, bar in ((torch.float32, 3e-5), (torch.bfloat16, 6e-2)):
        m = ms[dt]; cache = m.new_cache(2)                   # two slots for three requests: the pool grows
        slots = [cache.alloc() for _ in seqs]
        got = [[] for _ in seqs]
        lg = m.step(cache.begin_step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cuts)], [list(range(c)) for c in cuts]), cache)
        at = 0
        for i, c in enumerate(cuts):
            got[i].append(lg[at: at + c]); at += c
        pos = list(cuts); alive = [0, 1, 2]; late_slot = None; late_pos = 0; got_late = []
        while alive or (late_slot is not None and late_pos < len(late)):
            entries, who = [], []
            for i in alive:
                entries.append((slots[i], [seqs[i][pos[i]]])); who.append(i)
            if late_slot is not None and late_pos < len(late) and late_pos > 0:
                entries.append((late_slot, [late[late_pos]])); who.append("late")
            lg = m.step(cache.begin_step(entries, [[0]] * len(entries)), cache)
            for r, i in enumerate(who):
                if i == "late":
                    got_late.append(lg[r: r + 1]); late_pos += 1
                else:
                    got[i].append(lg[r: r + 1]); pos[i] += 1
            for i in list(alive):
                if pos[i] == len(seqs[i]):
                    alive.remove(i); cache.release(slots[i])
                    if late_slot is None:                    # the newcomer takes the slot that was just given back
                        late_slot = cache.alloc()
                        assert late_slot == slots[i]
                        lg = m.step(cache.begin_step([(late_slot, late[:7])], [list(range(7))]), cache)
                        got_late.append(lg); late_pos = 7
        for i in range(3):
            assert logit_err(torch.cat(got[i]), refs[i], QUANT[dt]) < bar, f"request {i} {dt}"
        assert logit_err(torch.cat(got_late), ref_late, QUANT[dt]) < bar, f"late request {dt}"
        assert cache.in_use() == 1


def test_long_prompt_at_odd_sizes_runs_the_segmented_and_matrix_core_paths(gpu, tmp_path):
    """A 600-token prompt beside a 70-token one through a model whose sizes are multiples of nothing convenient: the recurrent layers run in time segments,
    the bfloat16 attention on the matrix cores with scalar staging, the experts through the expert-sorted products; then both requests are decoded."""
    from exllamav3_amd.registry import load_model
    layers = [dict(type="gla", heads=3, dim=40, vdim=56, tau=5.0, rank=6, mlp=("moe", 36, 5, 2)),
              dict(type="attention", heads=6, kv_heads=2, dim=20, vdim=28, window=50, mlp=("dense", 150)),
              dict(type="gla", heads=1, dim=24, vdim=200, tau=30.0, rank=2, mlp=None)]
    cfg, t = mo.random_model(layers, vocab=300, width=88, seed=77)
    mo.save_model(str(tmp_path), cfg, t)
    orc = mo.OracleModel(cfg, t)
    seqs = [toks(300, 610, 5), toks(300, 80, 6)]
    cuts = [600, 70]
    refs = [orc.forward(s) for s in seqs]
    for dt, bar in ((torch.float32, 3e-5), (torch.bfloat16, 6e-2)):
        m = load_model(str(tmp_path), gpu, dt); cache = m.new_cache(2)
        slots = [cache.alloc(), cache.alloc()]
        want = [list(range(0, c, 7)) + [c - 1] for c in cuts]
        lg = m.step(cache.begin_step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cuts)], want), cache)
        got = [[lg[:len(want[0])]], [lg[len(want[0]):]]]
        rows = [list(want[0]), list(want[1])]
        for p in range(10):
            lg = m.step(cache.begin_step([(sl, [s[c + p]]) for sl, s, c in zip(slots, seqs, cuts)], [[0], [0]]), cache)
            for i in range(2):
                got[i].append(lg[i: i + 1]); rows[i].append(cuts[i] + p)
        for i in range(2):
            assert logit_err(torch.cat(got[i]), refs[i][rows[i]], QUANT[dt]) < bar, f"request {i} {dt}"


def test_long_decoding_stays_on_the_oracle(models):
    orc, ms, vocab = models["a"]
    t = toks(vocab, 140, 4)                                  # 4 prompt tokens, 136 decoded: the 6- and 33-token rings wrap many times
    ref = orc.forward(t)
    m = ms[torch.float32]; cache = m.new_cache(1); slot = cache.alloc()
    out = [m.step(cache.begin_step([(slot, t[:4])], [[0, 1, 2, 3]]), cache)]
    for p in range(4, len(t)):
        out.append(m.step(cache.begin_step([(slot, [t[p]])], [[0]]), cache))
    assert logit_err(torch.cat(out), ref) < 3e-5


def test_a_step_that_continues_a_sequence_by_several_tokens_is_refused(models):
    orc, ms, vocab = models["a"]
    m = ms[torch.float32]; cache = m.new_cache(1); slot = cache.alloc()
    m.step(cache.begin_step([(slot, [1, 2, 3])]), cache)
    with pytest.raises(RuntimeError):
        cache.begin_step([(slot, [4, 5])])


@pytest.mark.parametrize("name", ["a", "c"])
def test_greedy_generation_through_the_scheduler_matches_oracle(models, name):
    from exllamav3_amd.generator import Generator
    orc, ms, vocab = models[name]
    prompts = [toks(vocab, n, 50 + n) for n in (5, 17, 2, 11)]
    new = 12
    want = []
    for p in prompts:
        s = list(p)
        for _ in range(new):
            s.append(int(orc.forward(s)[-1].argmax()))
        want.append(s[len(p):])
    gen = Generator(ms[torch.float32], max_batch=3)          # four jobs, three at a time: the fourth is admitted into a freed slot while others decode
    got = gen.generate(prompts, max_new_tokens=new)
    assert got == want
    assert gen.cache.in_use() == 0


def test_decode_graphs_replay_bit_for_bit_what_eager_steps_compute(models):
    """The generator captures the decode step of a batch size the second time it occurs and replays it afterwards.  Two generators over the same
    jobs, one eager and one with graphs, are stepped side by side (so eager work and synchronisations lie between the replays): every step's
    sampled tokens are equal, and the logits of every replayed step equal the eager step's bit for bit.  Jobs end at different times, so several batch
    sizes are captured, and the moe layers' decode path (no host read) is inside the graph."""
    from exllamav3_amd.generator import Generator, Job
    orc, ms, vocab = models["c"]
    for dt in (torch.float32, torch.bfloat16):
        m = ms[dt]
        prompts = [toks(vocab, n, 70 + n) for n in (9, 4, 15)]
        lens = [30, 12, 21]
        ge, gg = Generator(m, cache=m.new_cache(4), graphs=False), Generator(m, cache=m.new_cache(4), graphs=True)
        seen = {"e": [], "g": []}
        for gen, key in ((ge, "e"), (gg, "g")):
            inner = gen._decode_step
            gen._decode_step = (lambda entries, inner=inner, key=key: seen[key].append(inner(entries).clone()) or seen[key][-1])
            for p, n in zip(prompts, lens):
                gen.enqueue(Job(list(p), n))
        while ge.busy() or gg.busy():
            a, b = ge.iterate(), gg.iterate()
            torch.cuda.synchronize()
            assert [t for _, t in a] == [t for _, t in b]
        assert gg.graph_replays >= 20 and len(gg._graphs) == 3 and ge.graph_replays == 0
        assert len(seen["e"]) == len(seen["g"])
        for x, y in zip(seen["e"], seen["g"]):
            assert torch.equal(x, y)


def test_trace_replay_writes_the_same_logits_however_the_tokens_are_cut(models, tmp_path):
    """TraceSession (what bin/trace_run runs): a request alone in one step, the same request as a prompt step plus single tokens, and the same
    request batched with another one; the files hold float32 [wanted, vocab] in the order of the entries and of their wanted places, and slots are
    given back at "end"."""
    import io, json
    import numpy as np
    from exllamav3_amd.trace import TraceSession
    orc, ms, vocab = models["c"]
    m = ms[torch.float32]
    a, b = toks(vocab, 19, 31), toks(vocab, 8, 32)
    want_a = [0, 5, 11, 17, 18]

    def run(name, steps):
        out = tmp_path / name
        out.mkdir()
        ts = TraceSession(m, str(out))
        log = io.StringIO()
        ts.run([json.dumps(s) for s in steps], out=log)
        assert log.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
        assert ts.cache.in_use() == 0
        return {int(f.name.split(".")[0]): np.fromfile(f, dtype="<f4").reshape(-1, vocab) for f in out.iterdir()}

    whole = run("whole", [{"step": 0, "entries": [{"id": "a", "tokens": a, "want": want_a}], "end": ["a"]}])
    assert list(whole) == [0] and whole[0].shape == (len(want_a), vocab)
    ref = orc.forward(a)[want_a].numpy()
    assert np.abs(whole[0] - ref).max() < 3e-5 * np.abs(ref).max() * 10
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": a[:12], "want": [0, 5, 11]}], "end": []}]
    for p in range(12, 19):
        steps.append({"step": p - 11, "entries": [{"id": "x", "tokens": [a[p]], "want": [0] if p in want_a else []}], "end": ["x"] if p == 18 else []})
    cut = run("decode", steps)
    assert sorted(cut) == [0, 6, 7]                          # steps without a wanted place write no file
    assert np.abs(np.concatenate([cut[0], cut[6], cut[7]]) - whole[0]).max() < 1e-4
    steps = [{"step": 0, "entries": [{"id": "b", "tokens": b[:3], "want": [2]}, {"id": "a", "tokens": a[:12], "want": [0, 5, 11]}], "end": []}]
    for p in range(7):
        e = [{"id": "a", "tokens": [a[12 + p]], "want": [0] if 12 + p in want_a else []}]
        if 3 + p < len(b):
            e.insert(0, {"id": "b", "tokens": [b[3 + p]], "want": [0] if 3 + p == 7 else []})
        steps.append({"step": p + 1, "entries": e, "end": (["b"] if 3 + p == 7 else []) + (["a"] if p == 6 else [])})
    tog = run("together", steps)
    assert np.abs(np.concatenate([tog[0][1:], tog[6], tog[7]]) - whole[0]).max() < 1e-4
    refb = orc.forward(b).numpy()
    assert np.abs(tog[0][0] - refb[2]).max() < 1e-3 and np.abs(tog[5][0] - refb[7]).max() < 1e-3


def test_a_cache_that_grows_under_captured_graphs_keeps_every_sequence(models):
    """One job decodes alone from a one-slot cache until its decode step is a captured graph; then two more jobs arrive, the pool doubles twice (its
    buffers move), the graphs are dropped and captured again -- and all three jobs still produce the oracle's greedy tokens."""
    from exllamav3_amd.generator import Generator, Job
    orc, ms, vocab = models["a"]
    m = ms[torch.float32]
    prompts = [toks(vocab, n, 90 + n) for n in (6, 3, 9)]
    new = 14
    want = []
    for p in prompts:
        s = list(p)
        for _ in range(new):
            s.append(int(orc.forward(s)[-1].argmax()))
        want.append(s[len(p):])
    gen = Generator(m, cache=m.new_cache(1), graphs=True)
    jobs = [gen.enqueue(Job(list(prompts[0]), new))]
    for _ in range(5):
        gen.iterate()
    assert gen.graph_replays >= 2 and gen.cache.capacity == 1
    jobs += [gen.enqueue(Job(list(p), new)) for p in prompts[1:]]
    while gen.busy():
        gen.iterate()
    assert gen.cache.capacity == 4
    assert [j.output for j in jobs] == want

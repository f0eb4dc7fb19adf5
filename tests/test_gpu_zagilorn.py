"""GPU tests of the Zagilorn design (csrc/mix_latent.hip, mix_rowops.hip, modules.py, zagilorn.py) against the float64 oracle of
tests/zagilorn_oracle.py: every mechanism alone, whole models of several small shapes (written to a checkpoint folder and loaded through the
registry), prefill against token-by-token decoding, unequal batches against each request alone, slots that are freed and used again, keys just
inside and just outside the window in prompts and in decoding, the first tokens, long decoding over a ring that wraps many times, and greedy
generation through the scheduler.  float32 runs are held to float32 rounding; bfloat16 runs to a loose bar (the oracle does not round)."""
import json
import math
import os
import pytest
import torch
import zagilorn_oracle as zo

pytestmark = pytest.mark.gpu
F64 = torch.float64
TOL = {torch.float32: 3e-5, torch.bfloat16: 4e-2}


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from exllamav3_amd import _lib
    _lib.mixlib()
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")
    return torch.device("cuda:0")


def rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).abs().max() / (b.abs().max() + 1e-30))


def mk(gpu, v):
    return torch.tensor(v, dtype=torch.int32, device=gpu)


def batch_tensors(gpu, lens, pos0=None, slots=None):
    pos0 = pos0 or [0] * len(lens)
    slots = slots or list(range(len(lens)))
    cu = [0]
    for l in lens: cu.append(cu[-1] + l)
    seq = [i for i, l in enumerate(lens) for _ in range(l)]
    pos = [pos0[i] + j for i, l in enumerate(lens) for j in range(l)]
    return mk(gpu, cu), mk(gpu, seq), mk(gpu, pos), mk(gpu, slots), mk(gpu, pos0), mk(gpu, [p + l for p, l in zip(pos0, lens)])


# ---- small random models ------------------------------------------------------------------------------------------------------------------------

def attn_layer(kind, heads, dim, rot_dim, vdim, rank, window, base=10000.0, dims=None, scaling=None, mlp=None):
    rot = {"base": base, "dims": rot_dim if dims is None else dims}
    if scaling:
        rot["scaling"] = scaling
    return {"type": kind, "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": 1.0 / math.sqrt(dim + rot_dim),
                                     "mask": {"size": window}, "rot": rot}, "mlp": mlp}


def moe(ff, experts, top, scale=1.5, limit=1.0, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared:
        d["shared"] = {"ff": shared[0], "limit": shared[1]}
    return d


YARN = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}


def config(layers, width=64, vocab=80, loop=None, side=8, logit_scale=0.7, eps=1e-5):
    c = {"architecture": "Zagilorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers, "logit_scale": logit_scale}
    if loop:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    if side:
        c["token_side"] = {"dim": side}
    return c


def weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    W, w = {}, cfg["width"]
    lin = lambda o, i, gain=1.0: (torch.randn(o, i, generator=g) * gain / math.sqrt(i))
    def norm(name):
        W[name] = 1.0 + 0.2 * torch.randn(w, generator=g); W[name + ".b"] = 0.1 * torch.randn(w, generator=g)
        W[name + ".alpha"] = torch.tensor(0.4 + 0.4 * float(torch.rand((), generator=g)))
    W["embed"] = torch.randn(cfg["vocab"], w, generator=g)
    W["head"] = lin(cfg["vocab"], w)
    norm("final.norm")
    if cfg.get("loop"):
        W["loop.in"] = lin(w, 2 * w, 1.4)
    sd = cfg.get("token_side", {}).get("dim", 0) if cfg.get("token_side") else 0
    if sd:
        W["side.embed"] = torch.randn(cfg["vocab"], sd * len(cfg["layers"]), generator=g)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        norm(p + "norm1")
        W[p + "mix.q"] = lin(H * (d + r), w, 2.0); W[p + "mix.dkv"] = lin(rank + r, w, 2.0)
        W[p + "mix.dkv.norm"] = 1.0 + 0.2 * torch.randn(rank, generator=g)
        W[p + "mix.uk"] = lin(H * d, rank, 2.0); W[p + "mix.uv"] = lin(H * dv, rank); W[p + "mix.o"] = lin(w, H * dv)
        if L["type"] == "latent_attention":
            W[p + "mix.sink"] = torch.randn(H, generator=g); W[p + "mix.g"] = lin(H * dv, w)
        f = L.get("mlp")
        if f:
            norm(p + "norm2")
            if f["kind"] == "dense":
                W[p + "mlp.up"] = lin(f["ff"], w); W[p + "mlp.down"] = lin(w, f["ff"])
            else:
                for e in range(f["router"]["experts"]):
                    W[f"{p}mlp.e{e}.gate"] = lin(f["expert"]["ff"], w, 2.0); W[f"{p}mlp.e{e}.up"] = lin(f["expert"]["ff"], w, 2.0); W[f"{p}mlp.e{e}.down"] = lin(w, f["expert"]["ff"])
                W[p + "mlp.router"] = lin(f["router"]["experts"], w, 2.0); W[p + "mlp.correction"] = 0.2 * torch.randn(f["router"]["experts"], generator=g)
                if f.get("shared"):
                    W[p + "mlp.shared.gate"] = lin(f["shared"]["ff"], w, 2.0); W[p + "mlp.shared.up"] = lin(f["shared"]["ff"], w, 2.0); W[p + "mlp.shared.down"] = lin(w, f["shared"]["ff"])
        if sd:
            W[p + "side.gate"] = lin(sd, w); W[p + "side.proj"] = lin(w, sd); W[p + "side.norm"] = 0.5 + 0.1 * torch.randn(w, generator=g)
    return {k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}


def save_and_load(tmp, cfg, W, gpu, dtype):
    from safetensors.torch import save_file
    from exllamav3_amd import registry
    os.makedirs(tmp, exist_ok=True)
    with open(os.path.join(tmp, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(W, os.path.join(tmp, "model.safetensors"))
    return registry.load_model(str(tmp), gpu, dtype)


# shapes chosen so that nothing the design allows happens to be equal or 1 by accident, and some things are: one head, top 1, every expert chosen,
# a window of one token, a window longer than any prompt, no feed-forward, no shared expert, fewer rotated dimensions than rot_dim, a loop that
# starts after the first layer, a loop of one pass, no loop, no token side input, sizes that are no multiple of 8
MODELS = {
    "loop_front": lambda: config([attn_layer("latent_attention_2", 2, 16, 8, 24, 32, 9, mlp={"kind": "dense", "ff": 96}),
                                  attn_layer("latent_attention", 3, 8, 8, 16, 24, 5, scaling=YARN, mlp=moe(16, 6, 2, shared=(24, 0.8))),
                                  attn_layer("latent_attention_2", 2, 16, 8, 8, 40, 12, mlp=moe(24, 4, 1, limit=0.5))], loop=(0, 2, 3)),
    "loop_middle": lambda: config([attn_layer("latent_attention", 1, 24, 16, 24, 16, 7, dims=8, scaling=YARN, mlp=None),
                                   attn_layer("latent_attention_2", 4, 8, 4, 8, 16, 1, mlp={"kind": "dense", "ff": 40}),
                                   attn_layer("latent_attention", 2, 12, 6, 10, 20, 300, mlp=moe(8, 3, 3, scale=1.0)),
                                   attn_layer("latent_attention_2", 2, 8, 8, 8, 8, 4, mlp={"kind": "dense", "ff": 32})], width=48, loop=(1, 3, 2), side=6, logit_scale=1.0),
    "no_loop_no_side": lambda: config([attn_layer("latent_attention", 2, 16, 8, 16, 24, 6, mlp=moe(16, 5, 2, shared=(16, 2.0))),
                                       attn_layer("latent_attention_2", 2, 16, 8, 16, 24, 11, base=500.0, mlp={"kind": "dense", "ff": 64})], side=0, logit_scale=2.5),
    "one_pass": lambda: config([attn_layer("latent_attention", 2, 8, 8, 8, 16, 8, scaling=YARN, mlp={"kind": "dense", "ff": 48})], width=40, loop=(0, 1, 1), side=4),
}


@pytest.fixture(scope="module")
def zoo(gpu, tmp_path_factory):
    """name -> (config, weights, {dtype: loaded model}); models are loaded once."""
    out = {}
    for k, (name, mkcfg) in enumerate(MODELS.items()):
        cfg = mkcfg()
        W = weights(cfg, 100 + k)
        d = tmp_path_factory.mktemp(name)
        out[name] = (cfg, W, {dt: save_and_load(str(d), cfg, W, gpu, dt) for dt in (torch.float32, torch.bfloat16)})
    return out


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def run_whole(model, cache, toks, want=None):
    s = cache.alloc()
    lg = model.step(cache.begin_step([(s, toks)], [want if want is not None else list(range(len(toks)))]), cache)
    cache.release(s)
    return lg.cpu()


# ---- mechanisms alone -----------------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_residual_update_and_dyn_tanh(gpu, dtype):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(3)
    n, w = 7, 100
    x0 = torch.randn(n, w, generator=g); wide = torch.randn(n, 2 * w + 3, generator=g).to(dtype)
    y = wide[:, 3: 3 + w]
    nw, nb, rw, alpha = torch.randn(w, generator=g), torch.randn(w, generator=g), torch.randn(w, generator=g), 0.37
    dev = lambda t: t.to(gpu)
    for mode in (mix_ops.RES_KEEP, mix_ops.RES_ADD, mix_ops.RES_SET):
        for rms in (False, True):
            for out in (mix_ops.OUT_NONE, mix_ops.OUT_CAST, mix_ops.OUT_DYN_TANH):
                if mode == mix_ops.RES_KEEP and (rms or out == mix_ops.OUT_NONE):
                    continue
                x = dev(x0.clone()); hbuf = torch.full((n, 2 * w), float("nan"), dtype=dtype, device=gpu); h = hbuf[:, w:]
                mix_ops.residual_norm(x, dev(wide)[:, 3: 3 + w], mode, dev(rw) if rms else None, 1e-5, out, alpha, dev(nw), dev(nb), h if out else None)
                yy = y.to(F64)
                if rms:
                    yy = zo.unit_rms(yy, 1e-5) * rw.to(F64)
                want_x = x0.to(F64) if mode == mix_ops.RES_KEEP else (x0.to(F64) + yy if mode == mix_ops.RES_ADD else yy)
                assert rel(x, want_x) < 1e-6, (mode, rms, out)
                if out == mix_ops.OUT_CAST:
                    assert rel(h, want_x) < TOL[dtype] / 4
                if out == mix_ops.OUT_DYN_TANH:
                    assert rel(h, zo.dyn_tanh(want_x, alpha, nw.to(F64), nb.to(F64))) < TOL[dtype] / 4
                if out:
                    assert torch.isnan(hbuf[:, :w]).all()                # the neighbouring column block is untouched
    rows = mk(gpu, [5, 0, 5])
    hw = torch.empty((3, w), dtype=dtype, device=gpu)
    mix_ops.dyn_tanh_rows(hw, dev(x0), rows, alpha, dev(nw), dev(nb))
    assert rel(hw, zo.dyn_tanh(x0.to(F64)[[5, 0, 5]], alpha, nw.to(F64), nb.to(F64))) < TOL[dtype] / 4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ff", [70, 72, 2056])                      # element by element, and 16 bytes per thread (one block, several blocks)
def test_activations_token_gate_heads_gate(gpu, dtype, ff):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(4)
    n = 9
    z = (3 * torch.randn(n, 2 * ff, generator=g)).to(dtype)
    a, b = z[:, :ff].to(F64), z[:, ff:].to(F64)
    zd = z.to(gpu)
    out = torch.empty((n, ff), dtype=dtype, device=gpu)
    mix_ops.act(out, zd[:, :ff], mix_ops.ACT_RELU2); assert rel(out, torch.relu(a) ** 2) < TOL[dtype] / 4
    mix_ops.act(out, zd[:, ff:], mix_ops.ACT_GELU_TANH); assert rel(out, zo.gelu_tanh(b)) < TOL[dtype] / 4
    mix_ops.glu_act(out, zd[:, :ff], zd[:, ff:], mix_ops.GLU_SILU); assert rel(out, a * torch.sigmoid(a) * b) < TOL[dtype] / 4
    for limit in (0.5, 7.0):
        mix_ops.glu_act(out, zd[:, :ff], zd[:, ff:], mix_ops.GLU_CLAMPED_SWISH, limit)
        gg, uu = a.clamp(max=limit), b.clamp(-limit, limit)
        assert rel(out, gg * torch.sigmoid(1.702 * gg) * (uu + 1)) < TOL[dtype] / 4
    table = torch.randn(11, 3 * 10, generator=g).to(dtype); toks = [3, 10, 0, 3, 7, 7, 1, 2, 9]
    gate = torch.randn(n, 10, generator=g).to(dtype)
    o = torch.empty((n, 10), dtype=dtype, device=gpu)
    mix_ops.token_gate(o, gate.to(gpu), table.to(gpu), 20, mk(gpu, toks))
    assert rel(o, zo.gelu_tanh(gate.to(F64)) * table.to(F64)[toks][:, 20:30]) < TOL[dtype] / 4
    H, dv = 3, 5
    av = torch.randn(H, n, dv, generator=g).to(dtype); gt = torch.randn(n, H * dv, generator=g).to(dtype)
    o = torch.empty((n, H * dv), dtype=dtype, device=gpu)
    mix_ops.heads_gate(o, av.to(gpu), dv, n * dv, gt.to(gpu), H, dv)                                  # head-major in, token-major out
    want = av.to(F64).transpose(0, 1).reshape(n, H * dv)
    assert rel(o, want * torch.sigmoid(gt.to(F64))) < TOL[dtype] / 4
    mix_ops.heads_gate(o, av.transpose(0, 1).contiguous().to(gpu), H * dv, dv, None, H, dv)
    assert rel(o, want) < 1e-6


def test_sigmoid_router(gpu):
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(5)
    for n, E, top in ((50, 9, 3), (4, 4, 4), (70, 17, 1)):
        z = 2 * torch.randn(n, E, generator=g); corr = torch.randn(E, generator=g)
        idx = torch.empty((n, top), dtype=torch.int32, device=gpu); wts = torch.empty((n, top), dtype=torch.float32, device=gpu)
        mix_ops.topk_sigmoid(idx, wts, z.to(gpu), corr.to(gpu), 2.5)
        ri, rw = zo.sigmoid_route(z.to(F64), corr.to(F64), top, 2.5)
        assert torch.equal(idx.cpu().long().sort(-1).values, ri.sort(-1).values)
        got = torch.zeros(n, E, dtype=F64).scatter_(1, idx.cpu().long(), wts.cpu().double()); ref = torch.zeros(n, E, dtype=F64).scatter_(1, ri, rw)
        assert rel(got, ref) < 1e-6
    # the correction moves the choice and not the weight: expert 0 has the largest score, expert 2 the largest corrected score
    z = torch.tensor([[3.0, 0.0, 1.0]]); corr = torch.tensor([-5.0, -5.0, 0.0])
    idx = torch.empty((1, 1), dtype=torch.int32, device=gpu); wts = torch.empty((1, 1), dtype=torch.float32, device=gpu)
    mix_ops.topk_sigmoid(idx, wts, z.to(gpu), corr.to(gpu), 3.0)
    assert int(idx[0, 0]) == 2 and abs(float(wts[0, 0]) - 3.0) < 1e-6                               # one chosen expert: s / s * scale


def absorbed_reference(q_lat, q_rot, ring_rows, scale, sink):
    """scores over cached rows [c | k_rot] with the query [q_lat | q_rot]; values = c."""
    rank = q_lat.shape[-1]
    s = (ring_rows @ torch.cat([q_lat, q_rot])) * scale
    m = s.max() if sink is None else torch.maximum(s.max(), sink)
    e = torch.exp(s - m)
    den = e.sum() + (torch.exp(sink - m) if sink is not None else 0.0)
    return (e / den) @ ring_rows[:, :rank]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,d,r,rank,W", [(2, 8, 8, 24, 5), (3, 16, 4, 130, 64), (1, 4, 16, 520, 300), (2, 8, 6, 37, 1), (3, 16, 16, 256, 64), (18, 8, 8, 136, 40),
                                          (2, 8, 64, 512, 70), (16, 8, 24, 104, 33)])
def test_latent_cache_kernels_window_edges(gpu, dtype, H, d, r, rank, W):
    """latent_prep + latent_decode alone, with one key made to stand out: the key that is W - 1 tokens back is seen, the one W back is not, in a
    ring that has wrapped; rows of the cache that a sequence has not written hold NaN and must not be read."""
    from exllamav3_amd import mix_ops
    from exllamav3_amd.modules import rotary_frequencies
    g = torch.Generator().manual_seed(rank + W)
    T = 2 * W + 7
    row = rank + r
    dims = r - (r % 2)
    freq, mag = rotary_frequencies(dims, 1000.0, None)
    norm_w = 1 + 0.1 * torch.randn(rank, generator=g)
    dkv = torch.randn(T, row, generator=g).to(dtype)
    q = torch.randn(T, H * (d + r), generator=g).to(dtype)
    # reference cache rows
    c = zo.unit_rms(dkv[:, :rank].to(F64), 1e-5) * norm_w.to(F64)
    cos, sin = zo.rotary_tables(torch.arange(T), dims, 1000.0) if dims else (None, None)
    kr = zo.rotate_pairs(dkv[:, rank:].to(F64), cos, sin, dims) if dims else dkv[:, rank:].to(F64)
    rows = torch.cat([c, kr], -1)
    qr = q.to(F64).reshape(T, H, d + r)[:, :, d:]
    qr = zo.rotate_pairs(qr, cos, sin, dims) if dims else qr
    n_slots, slot = 3, 2
    ring = torch.full((n_slots, W, row), float("nan"), dtype=dtype, device=gpu)
    sink = torch.randn(H, generator=g)
    # prompt step of T - 3 tokens, then three decode steps
    P = T - 3
    cu, seq, pos, sl, p0, la = batch_tensors(gpu, [P], slots=[slot])
    ckr = torch.empty((P, row), dtype=dtype, device=gpu)
    qd = q[:P].to(gpu).clone()
    mix_ops.latent_prep(ckr, ring, dkv[:P].to(gpu), norm_w.to(gpu), qd, seq, pos, sl, la, freq.to(gpu), mag, 1e-5, H, d, r, rank)
    assert rel(ckr, rows[:P]) < TOL[dtype]
    assert rel(qd.view(P, H, d + r)[:, :, d:], qr[:P]) < TOL[dtype]
    assert torch.equal(qd.view(P, H, d + r)[:, :, :d].cpu(), q[:P].view(P, H, d + r)[:, :, :d])          # the unrotated part passes untouched
    kfull = torch.zeros((P, H * (d + r)), dtype=dtype, device=gpu)
    mix_ops.latent_fill_k(kfull, ckr, H, d, r, rank)
    assert torch.equal(kfull.view(P, H, d + r)[:, :, d:], ckr[:, None, rank:].expand(P, H, r)) and float(kfull.view(P, H, d + r)[:, :, :d].abs().max()) == 0.0
    assert torch.isnan(ring[:slot]).all()
    for t in range(P, T):
        cu, seq, pos, sl, p0, la = batch_tensors(gpu, [1], pos0=[t], slots=[slot])
        ck1 = torch.empty((1, row), dtype=dtype, device=gpu)
        q1 = q[t: t + 1].to(gpu).clone()
        mix_ops.latent_prep(ck1, ring, dkv[t: t + 1].to(gpu), norm_w.to(gpu), q1, seq, pos, sl, la, freq.to(gpu), mag, 1e-5, H, d, r, rank)
        for edge in (t - W + 1, t - W):                       # the oldest key the window keeps / the newest it has dropped
            if edge < 0:
                continue
            # a latent query that points along that key's latent, large enough that its weight is all but 1 when it is seen
            q_lat = torch.randn(H, 1, rank, generator=g) * 0.1 + 4.0 * c[edge].float() / (c[edge].norm() ** 2).float() * rank ** 0.5
            q_lat = q_lat.to(dtype)
            o_lat = torch.full((H, 1, rank), float("nan"), dtype=dtype, device=gpu)
            kernels = [False, True] if mix_ops.latent_mfma_ok(dtype, rank, r) else [False]           # lane-per-key kernel, matrix-core kernel
            for sk in (None, sink):
                for mfma in kernels:
                    o_lat.fill_(float("nan"))
                    mix_ops.latent_decode(o_lat, q_lat.to(gpu), q1, ring, None if sk is None else sk.to(gpu), sl, la, d, r, 0.9, mfma=mfma)
                    lo = max(0, t - W + 1)
                    want = torch.stack([absorbed_reference(q_lat[h, 0].to(F64), qr[t, h], rows[lo: t + 1], 0.9, None if sk is None else sk[h].to(F64)) for h in range(H)])
                    assert rel(o_lat[:, 0], want) < TOL[dtype], (t, edge, sk is None, mfma)
                    if edge >= lo and W > 1 and sk is None:
                        assert rel(o_lat[:, 0], c[edge].expand(H, rank)) < 0.2          # the test's premise: that key dominates when it is inside
    assert torch.isnan(ring[:slot]).all() and not torch.isnan(ring[slot]).any()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind,H,d,r,dv,rank,W,dims,scaling,lens", [
    ("latent_attention", 3, 16, 8, 24, 32, 7, None, YARN, [19, 1, 8]), ("latent_attention_2", 2, 24, 16, 16, 48, 40, 8, None, [90, 33]),
    ("latent_attention", 1, 8, 8, 40, 16, 1, None, None, [5, 9]), ("latent_attention_2", 4, 32, 32, 32, 64, 100, None, YARN, [260]),
    ("latent_attention", 2, 10, 6, 12, 20, 500, None, YARN, [70, 64])])
def test_latent_attention_mixer(gpu, dtype, kind, H, d, r, dv, rank, W, dims, scaling, lens):
    """The mixer alone over a packed prompt step (lane-per-key and matrix-core prefill) and then decode steps of all sequences together."""
    from exllamav3_amd.modules import LatentAttention
    from exllamav3_amd.state_cache import SlotStateCache
    g = torch.Generator().manual_seed(H * 10 + W)
    width = 56
    L = attn_layer(kind, H, d, r, dv, rank, W, base=3000.0, dims=dims, scaling=scaling)
    m = L["mixer"]
    Wt = {}
    lin = lambda o, i, gain=1.0: (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(torch.bfloat16)
    Wt["q"] = lin(H * (d + r), width, 2); Wt["dkv"] = lin(rank + r, width, 2); Wt["dkv.norm"] = (1 + 0.2 * torch.randn(rank, generator=g)).to(torch.bfloat16)
    Wt["uk"] = lin(H * d, rank, 2); Wt["uv"] = lin(H * dv, rank); Wt["o"] = lin(width, H * dv)
    both = kind == "latent_attention"
    if both:
        Wt["sink"] = torch.randn(H, generator=g).to(torch.bfloat16); Wt["g"] = lin(H * dv, width)

    class Stc:
        def get_tensor(self, key, device="cpu"):
            return Wt[key]
    mixer = LatentAttention(width, H, d, r, dv, rank, m["scale"], W, 1e-5, m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"), sink=both, gate=both)
    mixer.load(Stc(), "", dtype, gpu)
    extra = min(2 * W + 3, 40)
    tot = [l + extra for l in lens]
    hs = [torch.randn(t, width, generator=g).to(dtype) for t in tot]
    W64 = {k: v.to(F64) for k, v in Wt.items()}
    ref = [zo.latent_attention(h.to(F64), W64, "", m, 1e-5, both) for h in hs]
    cache = SlotStateCache([mixer.state_specs()], gpu, slots=len(lens) + 1)
    cache.layers[0]["ring"].fill_(float("nan"))
    slots = [cache.alloc() for _ in lens][::-1]
    sb = cache.begin_step([(s, [0] * l) for s, l in zip(slots, lens)])
    y, _ = mixer.forward(torch.cat([h[:l] for h, l in zip(hs, lens)]).to(gpu), sb, cache.layers[0])
    assert rel(y, torch.cat([r_[:l] for r_, l in zip(ref, lens)])) < TOL[dtype]
    for s_ in range(extra):
        sb = cache.begin_step([(s, [0]) for s in slots])
        y, _ = mixer.forward(torch.stack([h[l + s_] for h, l in zip(hs, lens)]).to(gpu), sb, cache.layers[0])
        assert rel(y, torch.stack([r_[l + s_] for r_, l in zip(ref, lens)])) < TOL[dtype], s_


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [2, 17, 90])
def test_sigmoid_routed_clamped_experts(gpu, dtype, n):
    """The three row regimes of the experts (per (row, choice), expert-major, expert-sorted products) with the clamped activation and a shared expert."""
    from exllamav3_amd.modules import GatedMLP, SparseExperts
    from exllamav3_amd.state_cache import StepBatch
    g = torch.Generator().manual_seed(n)
    width, ff, E, top = 48, 24, 7, 3
    f = moe(ff, E, top, scale=1.7, limit=0.6, shared=(40, 0.9))
    Wt = {}
    lin = lambda o, i, gain=1.0: (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(torch.bfloat16)
    for e in range(E):
        Wt[f"e{e}.gate"] = lin(ff, width, 2); Wt[f"e{e}.up"] = lin(ff, width, 2); Wt[f"e{e}.down"] = lin(width, ff)
    Wt["router"] = lin(E, width, 3); Wt["correction"] = (0.3 * torch.randn(E, generator=g)).to(torch.bfloat16)
    Wt["shared.gate"] = lin(40, width, 2); Wt["shared.up"] = lin(40, width, 2); Wt["shared.down"] = lin(width, 40)

    class Stc:
        def get_tensor(self, key, device="cpu"):
            return Wt[key]
    mlp = SparseExperts(width, ff, E, top, router="sigmoid", router_bias=False, correction=True, route_scale=1.7, act="clamped_swish", limit=0.6,
                        shared=GatedMLP(width, 40, "clamped_swish", 0.9))
    mlp.load(Stc(), "", dtype, gpu)
    h = torch.randn(n, width, generator=g).to(dtype)
    sb = StepBatch(n=n, batch=1, decode=False, max_rows=n, tokens=None, cu=None, tok_seq=None, tok_pos=None, slots=None, pos0=None, len_after=None)
    y, _ = mlp.forward(h.to(gpu), sb)
    want = zo.sparse_mlp(h.to(F64), {k: v.to(F64) for k, v in Wt.items()}, "", f)
    assert rel(y, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_side_input(gpu, dtype):
    """The per-layer token input alone: gate on the stream, the layer's slice of the token's second embedding row, projection; and its RMS-normed update."""
    from exllamav3_amd import mix_ops
    from exllamav3_amd.modules import TokenSide, update_residual
    from exllamav3_amd.state_cache import StepBatch
    g = torch.Generator().manual_seed(11)
    width, dim, layers, layer, vocab, n = 72, 12, 3, 1, 30, 13
    lin = lambda o, i: (torch.randn(o, i, generator=g) / math.sqrt(i)).to(torch.bfloat16)
    Wt = {"l1.side.gate": lin(dim, width), "l1.side.proj": lin(width, dim), "l1.side.norm": (0.5 + 0.1 * torch.randn(width, generator=g)).to(torch.bfloat16),
          "side.embed": torch.randn(vocab, dim * layers, generator=g).to(torch.bfloat16)}

    class Stc:
        def get_tensor(self, key, device="cpu"):
            return Wt[key]
    side = TokenSide(width, dim, layer, 1e-5)
    side.load(Stc(), "l1.side.", Wt["side.embed"].to(dtype).to(gpu), dtype, gpu)
    toks = torch.randint(0, vocab, (n,), generator=g)
    x0 = torch.randn(n, width, generator=g)
    xc = x0.to(dtype)                                          # what the gate reads: the stream in the activation type
    sb = StepBatch(n=n, batch=1, decode=False, max_rows=n, tokens=toks.int().to(gpu), cu=None, tok_seq=None, tok_pos=None, slots=None, pos0=None, len_after=None)
    y = side.forward(xc.to(gpu), sb)
    x = x0.to(gpu).clone()
    update_residual(x, y, None, rms_w=side.norm_w, eps=1e-5)
    W64 = {k: v.to(F64) for k, v in Wt.items()}
    want = x0.to(F64) + zo.token_side(xc.to(F64), toks, W64, "l1.", layer, dim, 1e-5)
    assert rel(x - x0.to(gpu), want - x0.to(F64)) < TOL[dtype]


# ---- whole models ---------------------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("name", list(MODELS))
def test_prefill_and_every_layer_run_match_oracle(gpu, zoo, name):
    cfg, W, models = zoo[name]
    toks = tokens(cfg, 70, 1)
    taps = []
    ref = zo.forward(toks, W, cfg, taps)
    m = models[torch.float32]
    cache = m.new_cache()
    m.layer_taps = []
    got = run_whole(m, cache, toks)
    mine, m.layer_taps = m.layer_taps, None
    assert len(mine) == len(taps) == len(zo.layer_runs(cfg))
    for i, (a, b) in enumerate(zip(mine, taps)):
        assert rel(a, b) < TOL[torch.float32], f"residual after layer run {i}"
    assert rel(got, ref) < TOL[torch.float32]
    mb = models[torch.bfloat16]
    gb = run_whole(mb, mb.new_cache(), toks)
    e = (gb.double() - ref).abs().max(-1).values / ref.abs().max()
    assert float(e.median()) < 6e-2 and torch.isfinite(gb).all()


@pytest.mark.parametrize("name", list(MODELS))
def test_decode_token_by_token_and_first_tokens(gpu, zoo, name):
    """Prompts of 1, 2 and 41 tokens, then one token per step far past every window: the same logits as the whole sequence at once."""
    cfg, W, models = zoo[name]
    toks = tokens(cfg, 95, 2)
    ref = zo.forward(toks, W, cfg)
    m = models[torch.float32]
    whole = run_whole(m, m.new_cache(), toks)
    assert rel(whole, ref) < TOL[torch.float32]
    for P in (1, 2, 41):
        cache = m.new_cache()
        s = cache.alloc()
        got = [m.step(cache.begin_step([(s, toks[:P])], [list(range(P))]), cache).cpu()]
        for t in range(P, len(toks)):
            got.append(m.step(cache.begin_step([(s, [toks[t]])]), cache).cpu())
        assert rel(torch.cat(got), ref) < TOL[torch.float32], P
    mb = models[torch.bfloat16]
    cache = mb.new_cache(); s = cache.alloc()
    got = [mb.step(cache.begin_step([(s, toks[:30])], [list(range(30))]), cache).cpu()]
    for t in range(30, len(toks)):
        got.append(mb.step(cache.begin_step([(s, [toks[t]])]), cache).cpu())
    e = (torch.cat(got).double() - ref).abs().max(-1).values / ref.abs().max()
    assert float(e.median()) < 6e-2


@pytest.mark.parametrize("name", ["loop_front", "loop_middle"])
def test_unequal_batch_and_reused_slots(gpu, zoo, name):
    """Requests of unequal length in one packed step and decoded together, the shorter ones ending earlier, in slots that earlier requests used and
    that were filled with NaN in between: every request's logits equal those of the request alone."""
    cfg, W, models = zoo[name]
    m = models[torch.float32]
    lens, total = [1, 37, 14, 60], [9, 50, 40, 75]
    seqs = [tokens(cfg, t, 10 + i) for i, t in enumerate(total)]
    refs = [zo.forward(s, W, cfg) for s in seqs]
    cache = m.new_cache(slots=2)                              # grows while in use
    old = [cache.alloc() for _ in range(5)]
    m.step(cache.begin_step([(s, tokens(cfg, 20 + 3 * s, 50 + s)) for s in old]), cache)
    for s in (old[3], old[0], old[4], old[1]):
        cache.release(s)
    for layer in cache.layers:
        for buf in layer.values():
            for s in (old[3], old[0], old[4], old[1]):
                buf[s].fill_(float("nan"))
    slots = [cache.alloc() for _ in lens]
    assert set(slots) == {old[3], old[0], old[4], old[1]}
    got = [[] for _ in lens]
    lg = m.step(cache.begin_step([(s, q[:l]) for s, q, l in zip(slots, seqs, lens)], [list(range(l)) for l in lens]), cache).cpu()
    at = 0
    for i, l in enumerate(lens):
        got[i].append(lg[at: at + l]); at += l
    pos = list(lens)
    while any(p < t for p, t in zip(pos, total)):
        live = [i for i in range(len(lens)) if pos[i] < total[i]]
        lg = m.step(cache.begin_step([(slots[i], [seqs[i][pos[i]]]) for i in live]), cache).cpu()
        for k, i in enumerate(live):
            got[i].append(lg[k: k + 1]); pos[i] += 1
            if pos[i] == total[i]:
                cache.release(slots[i])
    for i in range(len(lens)):
        assert rel(torch.cat(got[i]), refs[i]) < TOL[torch.float32], i
    assert cache.in_use() == 1                                # old[2] still holds its sequence


def test_long_decoding_over_wrapped_rings(gpu, zoo):
    cfg, W, models = zoo["loop_front"]                         # windows 9, 5, 12: 160 decoded tokens wrap every ring many times
    toks = tokens(cfg, 170, 7)
    ref = zo.forward(toks, W, cfg)
    for dt in (torch.float32, torch.bfloat16):
        m = models[dt]
        cache = m.new_cache(); s = cache.alloc()
        got = [m.step(cache.begin_step([(s, toks[:10])], [list(range(10))]), cache).cpu()]
        for t in range(10, len(toks)):
            got.append(m.step(cache.begin_step([(s, [toks[t]])]), cache).cpu())
        e = (torch.cat(got).double() - ref).abs().max(-1).values / ref.abs().max()
        if dt == torch.float32:
            assert float(e.max()) < TOL[dt]
        else:
            assert float(e.median()) < 6e-2 and float(e[-20:].median()) < 6e-2


def test_matrix_core_prefill_long_prompt_bfloat16(gpu, zoo):
    """A prompt long enough for several 128-row blocks and 64-key tiles per window, in a batch with a short one."""
    cfg, W, models = zoo["loop_middle"]                        # one window of 300, one of 1
    seqs = [tokens(cfg, 420, 21), tokens(cfg, 33, 22)]
    refs = [zo.forward(s, W, cfg) for s in seqs]
    for dt in (torch.float32, torch.bfloat16):
        m = models[dt]
        cache = m.new_cache()
        sl = [cache.alloc(), cache.alloc()]
        lg = m.step(cache.begin_step(list(zip(sl, seqs)), [list(range(len(s))) for s in seqs]), cache).cpu()
        for got, ref in ((lg[:420], refs[0]), (lg[420:], refs[1])):
            e = (got.double() - ref).abs().max(-1).values / ref.abs().max()
            assert float(e.max()) < TOL[dt] if dt == torch.float32 else float(e.median()) < 6e-2


def test_a_step_that_continues_by_several_tokens_is_refused(gpu, zoo):
    cfg, W, models = zoo["one_pass"]
    m = models[torch.float32]
    cache = m.new_cache(); s = cache.alloc()
    m.step(cache.begin_step([(s, [1, 2, 3])]), cache)
    with pytest.raises(RuntimeError):
        cache.begin_step([(s, [4, 5])])


def test_window_edge_shows_in_the_logits(gpu, zoo):
    """Changing the token that lies exactly `window` back from the last one (outside every layer's reach through ONE layer run) must leave a one-layer
    model's last logits unchanged, and changing the one at window - 1 must change them: in a prompt and in decoding."""
    cfg, W, models = zoo["one_pass"]                           # one layer, one pass, window 8
    win = cfg["layers"][0]["mixer"]["mask"]["size"]
    m = models[torch.float32]
    base = tokens(cfg, 30, 5)
    def last_logits(toks, decode_from):
        cache = m.new_cache(); s = cache.alloc()
        lg = m.step(cache.begin_step([(s, toks[:decode_from])]), cache)
        for t in range(decode_from, len(toks)):
            lg = m.step(cache.begin_step([(s, [toks[t]])]), cache)
        return lg[0].cpu()
    for decode_from in (30, 12):
        ref = last_logits(base, decode_from)
        outside = list(base); outside[29 - win] = (outside[29 - win] + 1) % cfg["vocab"]
        inside = list(base); inside[29 - win + 1] = (inside[29 - win + 1] + 1) % cfg["vocab"]
        assert rel(last_logits(outside, decode_from), ref) < 1e-6
        assert rel(last_logits(inside, decode_from), ref) > 1e-4
        assert rel(last_logits(inside, decode_from), zo.forward(inside, W, cfg)[-1]) < TOL[torch.float32]


def test_greedy_generation_through_the_scheduler(gpu, zoo):
    from exllamav3_amd.generator import Generator
    cfg, W, models = zoo["loop_front"]
    m = models[torch.float32]
    prompts = [tokens(cfg, 5, 31), tokens(cfg, 23, 32), tokens(cfg, 1, 33)]
    want = [zo.greedy(p, 12, W, cfg) for p in prompts]
    for graphs in (False, True):
        gen = Generator(m, max_batch=2, graphs=graphs)        # the third prompt waits for a slot that a finished job gives back
        outs = gen.generate(prompts, max_new_tokens=12)
        assert outs == want, graphs
        assert gen.cache.in_use() == 0
        if graphs:
            assert gen.graph_replays > 0


def test_trace_replay_writes_the_wanted_logits(gpu, zoo, tmp_path):
    import io
    import numpy as np
    from exllamav3_amd.trace import TraceSession
    cfg, W, models = zoo["no_loop_no_side"]
    m = models[torch.float32]
    a, b = tokens(cfg, 12, 41), tokens(cfg, 5, 42)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [0, 8]}, {"id": "b", "tokens": b[:4], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[9:10], "want": [0]}, {"id": "b", "tokens": b[4:5], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[10:11], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[11:12], "want": [0]}], "end": ["a"]}]
    out = io.StringIO()
    sess = TraceSession(m, str(tmp_path))
    sess.run([json.dumps(s) for s in steps], out)
    assert out.getvalue().split() == ["done", "0", "done", "1", "done", "2", "done", "3"]
    ra, rb = zo.forward(a, W, cfg), zo.forward(b, W, cfg)
    rd = lambda k: torch.from_numpy(np.fromfile(os.path.join(str(tmp_path), f"{k}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]))
    assert rel(rd(0), ra[[0, 8]]) < TOL[torch.float32]
    assert rel(rd(1), torch.stack([ra[9], rb[4]])) < TOL[torch.float32]
    assert not os.path.exists(os.path.join(str(tmp_path), "2.f32"))
    assert rel(rd(3), ra[11:12]) < TOL[torch.float32]
    assert sess.cache.in_use() == 0


@pytest.mark.parametrize("H,r,rank,W,lens", [(5, 16, 64, 100, [3, 100, 57, 1]), (33, 8, 128, 300, [299, 301, 64]), (16, 64, 512, 129, [129, 40]), (4, 0, 200, 77, [500, 76])])
def test_matrix_core_latent_decode_batches_and_splits(gpu, H, r, rank, W, lens):
    """The matrix-core decode kernel over a batch of sequences of unequal length (shorter than, equal to and longer than the window, so rings are part
    filled, exactly full and wrapped), with every number of key splits from one to more than there are key tiles, against the float64 form."""
    from exllamav3_amd import mix_ops
    g = torch.Generator().manual_seed(rank + W)
    B, row, d = len(lens), rank + r, 8
    ring = torch.full((B + 2, W, row), float("nan"), dtype=torch.bfloat16, device=gpu)
    slots = [B + 1 - i for i in range(B)]
    rows = []
    for b, L in enumerate(lens):
        cnt = min(L, W)
        data = torch.randn(cnt, row, generator=g).to(torch.bfloat16)
        ring[slots[b], :cnt] = data.to(gpu)
        rows.append(data.to(F64))
    q_lat = (torch.randn(H, B, rank, generator=g) * 0.3).to(torch.bfloat16)
    q = torch.randn(B, H * (d + r), generator=g).to(torch.bfloat16)
    sink = torch.randn(H, generator=g)
    for sk in (None, sink, sink + 9.0):                       # no sink, one among the scores, one that takes most of the weight
        want = torch.stack([torch.stack([absorbed_reference(q_lat[h, b].to(F64), q[b].view(H, d + r)[h, d:].to(F64), rows[b], 0.2, None if sk is None else sk[h].to(F64))
                                         for b in range(B)]) for h in range(H)])
        for target in (1, 7, 64, 4096):
            mix_ops.LATENT_MFMA_TARGET_WAVES, keep = target, mix_ops.LATENT_MFMA_TARGET_WAVES
            try:
                o = torch.full((H, B, rank), float("nan"), dtype=torch.bfloat16, device=gpu)
                mix_ops.latent_decode(o, q_lat.to(gpu), q.to(gpu), ring, None if sk is None else sk.to(gpu), mk(gpu, slots), mk(gpu, lens), d, r, 0.2, mfma=True)
            finally:
                mix_ops.LATENT_MFMA_TARGET_WAVES = keep
            assert rel(o, want) < TOL[torch.bfloat16], (sk is None, target)

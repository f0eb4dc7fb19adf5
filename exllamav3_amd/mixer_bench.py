"""
`bench.py --mixer-family`: prefill and decode throughput of the unquantized mixer family (Vofanex layers with random weights) at sizes
that resemble real models' layers, beside the EXL3 Llama path at the same width / ff / head shape, and each new kernel alone against
its own roofline.  Prints one JSON line; the default workload of bench.py and its contract are untouched.

Rooflines: 2.5 PFLOP/s dense bfloat16 on the matrix cores, 157 TFLOP/s float32 on the vector units, 8 TB/s HBM.
"""
from __future__ import annotations
import json
import math
import time
import torch

PEAK_BF16, PEAK_F32, PEAK_HBM = 2.5e15, 157.3e12, 8.0e12

SIZES = {
    # width, ff, heads, kv_heads, head dim (the Llama shapes of the same name), window, gla heads x (dim, vdim), experts / top / expert ff
    "1b": dict(width=2048, ff=8192, heads=32, kv_heads=8, dim=64, window=1024, gla=(16, 64, 128), moe=(8, 2, 2048), llama="llama-3.2-1b"),
    "8b": dict(width=4096, ff=14336, heads=32, kv_heads=8, dim=128, window=1024, gla=(32, 64, 128), moe=(8, 2, 3584), llama="llama-3.1-8b"),
}
LAYER_KINDS = [("gla", "dense"), ("gla", "moe"), ("attention", "dense")]


class TensorDict:
    """In-memory stand-in for the checkpoint reader (get_tensor only): random weights never touch the disk."""

    def __init__(self, tensors):
        self.t = tensors

    def get_tensor(self, key, device="cpu", optional=False):
        return self.t[key]


def synth(size: dict, kinds, vocab=32000, seed=0, device="cuda:0"):
    g = torch.Generator(device=device).manual_seed(seed)
    w, t, layers = size["width"], {}, []

    def lin(name, o, i, s=1.0):
        t[name] = (torch.randn(o, i, generator=g, device=device) * (s / math.sqrt(i))).to(torch.bfloat16)

    def vec(name, n, mean=0.0, s=0.1):
        t[name] = (mean + s * torch.randn(n, generator=g, device=device)).to(torch.bfloat16)
    lin("embed", vocab, w, math.sqrt(w)); lin("head", vocab, w); vec("final.norm", w, 1.0)
    for i, (mix, ff) in enumerate(kinds):
        p = f"l{i}."
        vec(p + "norm1", w, 1.0); vec(p + "norm2", w, 1.0)
        for r in ("rg1", "rg2"):
            lin(p + r, w, w); vec(p + r + ".b", w, 1.0)
        if mix == "attention":
            H, G, d = size["heads"], size["kv_heads"], size["dim"]
            lin(p + "mix.q", H * d, w); lin(p + "mix.k", G * d, w); lin(p + "mix.v", G * d, w); lin(p + "mix.g", H, w); lin(p + "mix.o", w, H * d)
            for b, n in (("q", H * d), ("k", G * d), ("v", G * d)):
                vec(p + f"mix.{b}.b", n)
            vec(p + "mix.sink", H)
            mixer = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": d ** -0.5, "mask": {"size": size["window"]}}
        else:
            H, d, dv = size["gla"]
            lin(p + "mix.q", H * d, w); lin(p + "mix.k", H * d, w); lin(p + "mix.v", H * dv, w); lin(p + "mix.g", H * dv, w); lin(p + "mix.o", w, H * dv)
            lin(p + "mix.a1", 16, w); lin(p + "mix.a2", H * d, 16); vec(p + "mix.a2.b", H * d, 3.0, 1.0); vec(p + "mix.norm", dv, 1.0)
            mixer = {"heads": H, "dim": d, "vdim": dv, "tau": 16.0}
        if ff == "dense":
            lin(p + "mlp.up", size["ff"], w); lin(p + "mlp.down", w, size["ff"])
            t[p + "mlp.act"] = torch.tensor([0.5, 0.25, 0.125, 0.0], device=device).to(torch.bfloat16)
            mlp = {"kind": "dense", "ff": size["ff"]}
        else:
            E, top, eff = size["moe"]
            for e in range(E):
                lin(f"{p}mlp.e{e}.gate", eff, w); lin(f"{p}mlp.e{e}.up", eff, w); lin(f"{p}mlp.e{e}.down", w, eff)
            lin(p + "mlp.router", E, w); vec(p + "mlp.router.b", E)
            mlp = {"kind": "moe", "expert": {"ff": eff}, "router": {"experts": E, "top": top}}
        layers.append({"type": mix, "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Vofanex", "vocab": vocab, "width": w, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0}, "layers": layers}
    return cfg, TensorDict(t)


def _time(fn, n, warm=2):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n):
        fn()
    e1.record(); torch.cuda.synchronize()
    return e0.elapsed_time(e1) / n * 1e-3


def _make_vofanex(size, kind, reps, dev):
    from .vofanex import VofanexModel
    cfg, td = synth(size, [kind] * reps, device=dev)
    return VofanexModel(cfg, td, device=dev, dtype=torch.bfloat16)


def model_legs(size_name: str, prompt: int, ctx: int, steps: int, dev, kinds=None, make=_make_vofanex):
    """Per layer kind: prefill seconds per layer at `prompt` rows, decode seconds per layer at batch 1 and 16 after `ctx` tokens (eager, and batch 1 as a captured graph).
    make(size, kind, reps, dev) builds a step-interface model of `reps` layers of one kind."""
    size, out = SIZES[size_name], {}
    for kind in (kinds or LAYER_KINDS):
        reps = 2
        m = make(size, kind, reps, dev)
        cache = m.new_cache(16)
        toks = torch.randint(0, 32000, (prompt,)).tolist()
        slots = [cache.alloc() for _ in range(16)]

        def prefill():
            cache.length[slots[0]] = 0
            m.step(cache.begin_step([(slots[0], toks)]), cache)
        tp = _time(prefill, max(2, steps // 10))
        for s in slots:
            cache.length[s] = ctx
        leg = {"prefill_ms_per_layer": tp / reps * 1e3, "prefill_tok_s_per_layer": prompt * reps / tp}
        for bs in (1, 16):
            def decode():
                for s in slots[:bs]:
                    cache.length[s] = ctx
                m.step(cache.begin_step([(s, [7 + 101 * i]) for i, s in enumerate(slots[:bs])]), cache)       # different tokens: the rows route differently
            leg[f"decode_bs{bs}_ms_per_layer"] = _time(decode, steps) / reps * 1e3
        # the same batch-1 step as one captured graph (replayed at a fixed position): what the launches cost
        for s in slots[:1]:
            cache.length[s] = ctx
        sb = cache.begin_step([(slots[0], [7])])
        st = torch.cuda.Stream()
        st.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(st):
            m.step(sb, cache)
        torch.cuda.current_stream().wait_stream(st); torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            m.step(sb, cache)
        leg["decode_bs1_graph_ms_per_layer"] = _time(gr.replay, steps) / reps * 1e3
        out["+".join(kind)] = leg
        del m, cache, gr
        torch.cuda.empty_cache()
    return out


def llama_legs(size_name: str, prompt: int, ctx: int, steps: int, dev):
    """The closest existing model: the EXL3 4-bit Llama layer of the same width / ff / heads (quantized linears, rope, 4-bit cache, float16)."""
    from . import ext
    from .llama_path import SHAPES, SyntheticEXL3Llama
    from .tp import TPBackendRCCL
    ext.init(dev.index)
    layers = 2
    m = SyntheticEXL3Llama(SHAPES[SIZES[size_name]["llama"]], K=4, cb=2, device=dev, backend=TPBackendRCCL(0, 1, dev), kv_bits=4, layers=layers, max_ctx=max(ctx + 64, prompt))
    out = {}
    m.alloc_state(1, pos=ctx)
    m.with_attention = True; m.prefill_attention = True
    out["decode_bs1_ms_per_layer"] = _time(m.decode_step_fx, steps) / layers * 1e3
    tp = _time(lambda: m.prefill_chunk(prompt), max(2, steps // 10))
    out["prefill_ms_per_layer"] = tp / layers * 1e3
    m.alloc_state(16, pos=ctx)
    out["decode_bs16_ms_per_layer"] = _time(m.decode_step_fx, steps) / layers * 1e3
    return out


def kernel_legs(size_name: str, prompt: int, ctx: int, dev):
    """Each new kernel alone at the size's shapes: seconds, and the fraction of the roofline that bounds it."""
    from . import mix_ops
    s = SIZES[size_name]
    out, bf = {}, torch.bfloat16
    rnd = lambda *sh: torch.randn(*sh, device=dev).to(bf)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    H, G, d, W = s["heads"], s["kv_heads"], s["dim"], s["window"]
    n = prompt
    cu, seq, pos = i32([0, n]), torch.zeros(n, dtype=torch.int32, device=dev), torch.arange(n, dtype=torch.int32, device=dev)
    sl, la, p0 = i32([0]), i32([n]), i32([0])
    q, k, v, gt, sink = rnd(n, H * d), rnd(n, G * d), rnd(n, G * d), rnd(n, H), torch.zeros(H, device=dev)
    rk, rv = torch.zeros((16, W, G, d), dtype=bf, device=dev), torch.zeros((16, W, G, d), dtype=bf, device=dev)
    vn, o = torch.empty((n, G, d), dtype=bf, device=dev), torch.empty((n, H * d), dtype=bf, device=dev)
    mix_ops.attn_store(vn, rk, rv, k, v, seq, pos, sl, la, 1e-5)
    t = _time(lambda: mix_ops.attn_prefill(o, q, k, vn, gt, sink, cu, seq, pos, H, d ** -0.5, W, max_rows=n, mfma=True), 10)
    pairs = sum(min(i + 1, W) for i in range(n))
    fl = 4.0 * d * pairs * H
    out["attn_prefill_mfma"] = {"ms": t * 1e3, "tflops": fl / t / 1e12, "of_bf16_peak": fl / t / PEAK_BF16}
    for bs in (1, 16):
        qd, gd, od = rnd(bs, H * d), rnd(bs, H), torch.empty((bs, H * d), dtype=bf, device=dev)
        sld, lad = torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx] * bs)
        t = _time(lambda: mix_ops.attn_decode(od, qd, rk, rv, gd, sink, sld, lad, H, d ** -0.5), 50)
        by = bs * min(ctx, W) * G * d * 2 * 2
        out[f"attn_decode_bs{bs}"] = {"us": t * 1e6, "GBps": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    Hg, dg, dvg = s["gla"]
    qg, kg, vg, gg, lr = rnd(n, Hg * dg), rnd(n, Hg * dg) * 0.3, rnd(n, Hg * dvg), rnd(n, Hg * dvg), rnd(n, 16)
    a2, a2b = rnd(Hg * dg, 16), torch.full((Hg * dg,), 3.0, device=dev)
    state = torch.zeros((16, Hg, dg, dvg), device=dev); og = torch.empty((n, Hg, dvg), device=dev)
    from .modules import GatedLinearAttention
    gl = GatedLinearAttention(s["width"], Hg, dg, dvg, 16.0, 1e-5)
    from .state_cache import StepBatch
    segs = gl.segments(StepBatch(n, 1, False, n, None, cu, seq, pos, sl, p0, la))
    fl = 4.0 * dg * dvg * Hg * n
    for name, sg in (("gla_prefill_segmented", segs), ("gla_prefill_one_chain", None)):
        t = _time(lambda: mix_ops.gla_scan(og, state, qg, kg, vg, lr, a2, a2b, cu, sl, p0, 16.0, dg ** -0.5, segments=sg), 5)
        out[name] = {"ms": t * 1e3, "segments": sg, "tflops_useful": fl / t / 1e12, "of_f32_vector_peak": fl / t / PEAK_F32}
    for bs in (1, 16):
        cud, sld, p0d = torch.arange(bs + 1, dtype=torch.int32, device=dev), torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx] * bs)
        ogd = torch.empty((bs, Hg, dvg), device=dev)
        t = _time(lambda: mix_ops.gla_scan(ogd, state, qg[:bs], kg[:bs], vg[:bs], lr[:bs], a2, a2b, cud, sld, p0d, 16.0, dg ** -0.5), 50)
        by = bs * Hg * dg * dvg * 4 * 2
        out[f"gla_decode_bs{bs}"] = {"us": t * 1e6, "GBps": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    w, ff = s["width"], s["ff"]
    x, y, r, nw, h = torch.randn(n, w, device=dev), rnd(n, w), rnd(n, w), torch.ones(w, device=dev), torch.empty((n, w), dtype=bf, device=dev)
    t = _time(lambda: mix_ops.gated_residual(x, y, r, nw, h, 1e-5), 20)
    by = n * w * (4 + 4 + 2 + 2 + 2)
    out["gated_residual_norm"] = {"us": t * 1e6, "GBps": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    z, a, coef = rnd(n, ff), torch.empty((n, ff), dtype=bf, device=dev), torch.tensor([0.5, 0.25, 0.125, 0.0], device=dev)
    t = _time(lambda: mix_ops.polynorm(a, z, coef, 1e-5), 20)
    by = n * ff * (2 + 2)
    out["polynorm"] = {"us": t * 1e6, "GBps": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    E, top, eff = s["moe"]
    wg, wu, wd = rnd(E, eff, w), rnd(E, eff, w), rnd(E, w, eff)
    for bs in (1, 16):
        hh, idx = rnd(bs, w), torch.stack([torch.randperm(E, device=dev)[:top] for _ in range(bs)]).int().contiguous()
        wt, hid, yy = torch.full((bs, top), 1.0 / top, device=dev), torch.empty((bs * top, eff), dtype=bf, device=dev), torch.empty((bs, w), dtype=bf, device=dev)

        def moe():
            mix_ops.moe_gate_up(hid, hh, wg, wu, idx); mix_ops.moe_down(yy, hid, wd, idx, wt)
        if bs > 1:
            def moe():
                mix_ops.moe_expert_major(yy, hh, wg, wu, wd, idx, wt)
        t = _time(moe, 50)
        by = min(bs * top, E) * 3 * eff * w * 2 if bs > 1 else top * 3 * eff * w * 2
        out[f"moe_decode_bs{bs}"] = {"us": t * 1e6, "GBps_distinct_weights": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    return out


def like_kernels(size_name: str, prompt: int, dev):
    """The like kernel of the closest model: the Llama path's prefill attention (float16, causal, no window) at the same head shape."""
    from . import ext
    s = SIZES[size_name]
    H, G, d = s["heads"], s["kv_heads"], s["dim"]
    page = 256
    pages = (prompt + page - 1) // page
    q = torch.randn(1, prompt, H, d, device=dev).half(); out = torch.empty_like(q)
    kp = torch.randn(pages, page, G, d, device=dev).half(); vp = torch.randn(pages, page, G, d, device=dev).half()
    bt = torch.arange(pages, dtype=torch.int32, device=dev).view(1, pages); ls = torch.tensor([prompt], dtype=torch.int32, device=dev)
    t = _time(lambda: ext.attn_prefill_paged(q, out, kp, vp, bt, ls), 10)
    fl = 4.0 * d * H * prompt * (prompt + 1) / 2
    return {"exl3_attn_prefill": {"ms": t * 1e3, "tflops": fl / t / 1e12, "of_f16_peak": fl / t / PEAK_BF16}}


def run(args) -> int:
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    from . import _lib
    _lib.mixlib()
    prompt, ctx = args.prefill_tokens, 1000
    res = {"metric": "mixer_family_layer_times", "unit": "ms per layer", "dtype": "bf16", "data": "synthetic", "prompt": prompt, "ctx": ctx, "sizes": {}}
    for name in (args.mixer_sizes.split(",") if args.mixer_sizes else list(SIZES)):
        t0 = time.time()
        entry = {"vofanex_layers": model_legs(name, prompt, ctx, args.steps, dev), "kernels": kernel_legs(name, prompt, ctx, dev)}
        try:
            entry["closest_model_exl3_llama_layer"] = llama_legs(name, prompt, ctx, args.steps, dev)
            entry["closest_model_kernels"] = like_kernels(name, prompt, dev)
        except Exception as e:                       # the comparison leg must not hide the new design's numbers
            entry["closest_model_error"] = f"{type(e).__name__}: {e}"
        entry["seconds"] = round(time.time() - t0, 1)
        res["sizes"][name] = entry
    print(json.dumps(res))
    return 0

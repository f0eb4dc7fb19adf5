"""
`bench.py --latent-family`: prefill and decode throughput of Zagilorn layers (latent attention with a relu^2 feed-forward or sigmoid-routed clamped experts,
Dynamic Tanh, token side input; random weights) at sizes that resemble real models' layers, beside the closest existing model -- Vofanex layers
(sliding-window sink attention with PolyNorm feed-forward or softmax-routed experts) of the same width / ff / expert shape, timed in the same process --
and each kernel of the design alone against its roofline, next to the like kernel of the closest model.  Prints one JSON line; the default workload of
bench.py and the JSON line it prints are untouched.
"""
from __future__ import annotations
import json
import math
import time
import torch
from .mixer_bench import PEAK_BF16, PEAK_HBM, SIZES, TensorDict, _time, kernel_legs, model_legs

# latent attention at the sizes of mixer_bench.SIZES: heads x (unrotated + rotated) query/key dims, value dim, latent rank; side input dim
LATENT = {
    "1b": dict(heads=16, dim=128, rot_dim=64, vdim=128, rank=512, side=256, shared_ff=2048),
    "8b": dict(heads=32, dim=128, rot_dim=64, vdim=128, rank=512, side=256, shared_ff=3584),
}
KINDS = [("latent_attention_2", "dense"), ("latent_attention", "moe")]
YARN = {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}


def synth(size: dict, lt: dict, kinds, vocab=32000, seed=0, device="cuda:0", loop=None):
    """Random Zagilorn weights and their config: size = width / ff / window / moe (experts, top, expert ff), lt = the latent-attention shape; loop = (start, stop, times)."""
    g = torch.Generator(device=device).manual_seed(seed)
    w, t, layers = size["width"], {}, []

    def lin(name, o, i, s=1.0):
        t[name] = (torch.randn(o, i, generator=g, device=device) * (s / math.sqrt(i))).to(torch.bfloat16)

    def vec(name, n, mean=0.0, s=0.1):
        t[name] = (mean + s * torch.randn(n, generator=g, device=device)).to(torch.bfloat16)

    def norm(name):
        vec(name, w, 1.0); vec(name + ".b", w); t[name + ".alpha"] = torch.tensor(0.5, device=device).to(torch.bfloat16)
    lin("embed", vocab, w, math.sqrt(w)); lin("head", vocab, w); norm("final.norm")
    lin("side.embed", vocab, lt["side"] * len(kinds), math.sqrt(lt["side"] * len(kinds)))
    H, d, r, dv, rank = lt["heads"], lt["dim"], lt["rot_dim"], lt["vdim"], lt["rank"]
    for i, (mix, ff) in enumerate(kinds):
        p = f"l{i}."
        norm(p + "norm1"); norm(p + "norm2")
        lin(p + "mix.q", H * (d + r), w); lin(p + "mix.dkv", rank + r, w); vec(p + "mix.dkv.norm", rank, 1.0)
        lin(p + "mix.uk", H * d, rank); lin(p + "mix.uv", H * dv, rank); lin(p + "mix.o", w, H * dv)
        rot = {"base": 10000.0, "dims": r}
        if mix == "latent_attention":
            vec(p + "mix.sink", H); lin(p + "mix.g", H * dv, w); rot["scaling"] = YARN
        mixer = {"heads": H, "dim": d, "rot_dim": r, "vdim": dv, "kv_rank": rank, "scale": (d + r) ** -0.5, "mask": {"size": size["window"]}, "rot": rot}
        if ff == "dense":
            lin(p + "mlp.up", size["ff"], w); lin(p + "mlp.down", w, size["ff"])
            mlp = {"kind": "dense", "ff": size["ff"]}
        else:
            E, top, eff = size["moe"]
            for e in range(E):
                lin(f"{p}mlp.e{e}.gate", eff, w); lin(f"{p}mlp.e{e}.up", eff, w); lin(f"{p}mlp.e{e}.down", w, eff)
            lin(p + "mlp.router", E, w); vec(p + "mlp.correction", E)
            lin(p + "mlp.shared.gate", lt["shared_ff"], w); lin(p + "mlp.shared.up", lt["shared_ff"], w); lin(p + "mlp.shared.down", w, lt["shared_ff"])
            mlp = {"kind": "moe", "expert": {"ff": eff, "limit": 7.0}, "router": {"experts": E, "top": top, "scale": 1.0}, "shared": {"ff": lt["shared_ff"], "limit": 7.0}}
        lin(p + "side.gate", lt["side"], w); lin(p + "side.proj", w, lt["side"]); vec(p + "side.norm", w, 1.0)
        layers.append({"type": mix, "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Zagilorn", "vocab": vocab, "width": w, "norm": {"eps": 1e-5}, "logit_scale": 1.0, "token_side": {"dim": lt["side"]}, "layers": layers}
    if loop:
        lin("loop.in", w, 2 * w, 1.4)
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg, TensorDict(t)


def _make(size_name):
    def make(size, kind, reps, dev):
        from .zagilorn import ZagilornModel
        cfg, td = synth(size, LATENT[size_name], [kind] * reps, device=dev)
        return ZagilornModel(cfg, td, device=dev, dtype=torch.bfloat16)
    return make


def latent_kernel_legs(size_name: str, prompt: int, ctx: int, dev):
    """Each kernel of the design alone at the size's shapes: time and the fraction of the roofline that bounds it."""
    from . import mix_ops
    from .modules import rotary_frequencies
    s, lt = SIZES[size_name], LATENT[size_name]
    out, bf = {}, torch.bfloat16
    rnd = lambda *sh: torch.randn(*sh, device=dev).to(bf)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    H, d, r, dv, rank, W, w, ff = lt["heads"], lt["dim"], lt["rot_dim"], lt["vdim"], lt["rank"], s["window"], s["width"], s["ff"]
    n, row, dk = prompt, lt["rank"] + lt["rot_dim"], lt["dim"] + lt["rot_dim"]
    cu, seq, pos = i32([0, n]), torch.zeros(n, dtype=torch.int32, device=dev), torch.arange(n, dtype=torch.int32, device=dev)
    sl, la = i32([0]), i32([n])
    hbm = lambda by, t: {"us": t * 1e6, "GBps": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    freq, mag = rotary_frequencies(r, 10000.0, YARN)
    freq = freq.to(dev)
    ring, ckr = torch.zeros((16, W, row), dtype=bf, device=dev), torch.empty((n, row), dtype=bf, device=dev)
    dkv, q, nw = rnd(n, row), rnd(n, H * dk), torch.ones(rank, device=dev)
    t = _time(lambda: mix_ops.latent_prep(ckr, ring, dkv, nw, q, seq, pos, sl, la, freq, mag, 1e-5, H, d, r, rank), 20)
    out["latent_prep_prefill"] = hbm(n * (row * 2 * 2 + H * r * 2 * 2) + W * row * 2, t)
    k, v, o = rnd(n, H * dk), rnd(n, H, dv), torch.empty((n, H * dv), dtype=bf, device=dev)
    t = _time(lambda: mix_ops.latent_fill_k(k, ckr, H, d, r, rank), 20)
    out["latent_fill_k"] = hbm(n * (r * 2 + H * r * 2), t)
    sink = torch.zeros(H, device=dev)
    t = _time(lambda: mix_ops.attn_prefill(o, q, k, v, None, sink, cu, seq, pos, H, dk ** -0.5, W, max_rows=n, mfma=True), 10)
    pairs = sum(min(i + 1, W) for i in range(n))
    fl = 2.0 * (dk + dv) * pairs * H
    out["attn_prefill_mfma_latent_shapes"] = {"ms": t * 1e3, "tflops": fl / t / 1e12, "of_bf16_peak": fl / t / PEAK_BF16}
    g = rnd(n, H * dv); o2 = torch.empty_like(o)
    t = _time(lambda: mix_ops.heads_gate(o2, o, H * dv, dv, g, H, dv), 20)
    out["heads_gate"] = hbm(n * H * dv * 2 * 3, t)
    for bs in (1, 16):
        qd, ql, ol = rnd(bs, H * dk), rnd(H, bs, rank), torch.empty((H, bs, rank), dtype=bf, device=dev)
        sld, lad = torch.arange(bs, dtype=torch.int32, device=dev), i32([ctx] * bs)
        t = _time(lambda: mix_ops.latent_decode(ol, ql, qd, ring, sink, sld, lad, d, r, dk ** -0.5), 50)
        by = bs * min(ctx, W) * row * 2                      # every cached row once per sequence
        e = hbm(by, t)
        e["tflops"] = bs * H * min(ctx, W) * (row + rank) * 2.0 / t / 1e12
        out[f"latent_decode_bs{bs}"] = e
        dkd, ck1, pd, sq = rnd(bs, row), torch.empty((bs, row), dtype=bf, device=dev), i32([ctx - 1] * bs), torch.arange(bs, dtype=torch.int32, device=dev)
        t = _time(lambda: mix_ops.latent_prep(ck1, ring, dkd, nw, qd, sq, pd, sld, lad, freq, mag, 1e-5, H, d, r, rank), 50)
        out[f"latent_prep_bs{bs}"] = {"us": t * 1e6}
    x, y, nb, h = torch.randn(n, w, device=dev), rnd(n, w), torch.zeros(w, device=dev), torch.empty((n, w), dtype=bf, device=dev)
    nw2 = torch.ones(w, device=dev)
    t = _time(lambda: mix_ops.residual_norm(x, y, mix_ops.RES_ADD, None, 0.0, mix_ops.OUT_DYN_TANH, 0.5, nw2, nb, h), 20)
    out["residual_dyn_tanh"] = hbm(n * w * (4 + 4 + 2 + 2), t)
    t = _time(lambda: mix_ops.residual_norm(x, y, mix_ops.RES_ADD, nw2, 1e-5, mix_ops.OUT_DYN_TANH, 0.5, nw2, nb, h), 20)
    out["residual_rms_addend_dyn_tanh"] = hbm(n * w * (4 + 4 + 2 + 2), t)
    z, a = rnd(n, ff), torch.empty((n, ff), dtype=bf, device=dev)
    t = _time(lambda: mix_ops.act(a, z, mix_ops.ACT_RELU2), 20)
    out["relu2"] = hbm(n * ff * 4, t)
    eff = s["moe"][2]
    gu, a2 = rnd(n, 2 * eff), torch.empty((n, eff), dtype=bf, device=dev)
    t = _time(lambda: mix_ops.glu_act(a2, gu[:, :eff], gu[:, eff:], mix_ops.GLU_CLAMPED_SWISH, 7.0), 20)
    out["clamped_swish_glu"] = hbm(n * eff * 6, t)
    sd = lt["side"]
    tb, gt, tg, tk = rnd(32000, sd * 2), rnd(n, sd), torch.empty((n, sd), dtype=bf, device=dev), torch.randint(0, 32000, (n,), device=dev).int()
    t = _time(lambda: mix_ops.token_gate(tg, gt, tb, sd, tk), 20)
    out["token_gate"] = hbm(n * sd * 6, t)
    lg, idx, wt, corr = torch.randn(n, s["moe"][0], device=dev), torch.empty((n, s["moe"][1]), dtype=torch.int32, device=dev), torch.empty((n, s["moe"][1]), device=dev), torch.zeros(s["moe"][0], device=dev)
    t = _time(lambda: mix_ops.topk_sigmoid(idx, wt, lg, corr, 1.0), 20)
    out["topk_sigmoid"] = {"us": t * 1e6}
    E, top, _ = s["moe"]
    wg, wu, wd = rnd(E, eff, w), rnd(E, eff, w), rnd(E, w, eff)
    for bs in (1, 16):
        hh, ix = rnd(bs, w), torch.stack([torch.randperm(E, device=dev)[:top] for _ in range(bs)]).int().contiguous()
        wts, hid, yy = torch.full((bs, top), 1.0 / top, device=dev), torch.empty((bs * top, eff), dtype=bf, device=dev), torch.empty((bs, w), dtype=bf, device=dev)
        if bs == 1:
            def moe():
                mix_ops.moe_gate_up_act(hid, hh, wg, wu, ix, mix_ops.GLU_CLAMPED_SWISH, 7.0); mix_ops.moe_down(yy, hid, wd, ix, wts)
        else:
            def moe():
                mix_ops.moe_expert_major(yy, hh, wg, wu, wd, ix, wts, mix_ops.GLU_CLAMPED_SWISH, 7.0)
        t = _time(moe, 50)
        by = min(bs * top, E) * 3 * eff * w * 2
        out[f"moe_clamped_decode_bs{bs}"] = {"us": t * 1e6, "GBps_distinct_weights": by / t / 1e9, "of_hbm": by / t / PEAK_HBM}
    return out


def run(args) -> int:
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    from . import _lib
    _lib.mixlib()
    prompt, ctx = args.prefill_tokens, 1000
    res = {"metric": "latent_family_layer_times", "unit": "ms per layer", "dtype": "bf16", "data": "synthetic", "prompt": prompt, "ctx": ctx, "sizes": {}}
    for name in (args.mixer_sizes.split(",") if args.mixer_sizes else list(SIZES)):
        t0 = time.time()
        entry = {"latent": LATENT[name], "zagilorn_layers": model_legs(name, prompt, ctx, args.steps, dev, kinds=KINDS, make=_make(name)),
                 "kernels": latent_kernel_legs(name, prompt, ctx, dev)}
        try:
            entry["closest_model_vofanex_layers"] = model_legs(name, prompt, ctx, args.steps, dev, kinds=[("attention", "dense"), ("attention", "moe")])
            entry["closest_model_kernels"] = kernel_legs(name, prompt, ctx, dev)
        except Exception as e:                       # the comparison leg must not hide the new design's numbers
            entry["closest_model_error"] = f"{type(e).__name__}: {e}"
        entry["seconds"] = round(time.time() - t0, 1)
        res["sizes"][name] = entry
    print(json.dumps(res))
    return 0

"""Slow float64 restatement of the mixer-family mechanisms, one function per mechanism, written from their equations and sharing no code
with exllamav3_amd (test infrastructure only).  Inputs are torch tensors; weights are used at the values stored in the checkpoint."""
import math
import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def sliding_sink_attention(q, k, v, scale, window, sink=None, gate=None, eps=1e-5, value_norm=True):
    """q [T,H,d], k [T,G,d], v [T,G,dv]; sink [H] or None; gate [T,H] pre-sigmoid or None.  Token i sees j with 0 <= i-j < window."""
    T, H, d = q.shape
    G = k.shape[1]
    if value_norm:
        v = unit_rms(v, eps)
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = max(0, i - window + 1)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            m = s.max() if sink is None else torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink[h] - m) if sink is not None else 0.0)
            out[i, h] = (e / den) @ v[lo:i + 1, g]
    if gate is not None:
        out = out * torch.sigmoid(gate)[:, :, None]
    return out


def gla_recurrent(q, k, v, z, tau, S0=None):
    """q,k,z [T,H,d], v [T,H,dv]; alpha = sigmoid(z)^(1/tau); S <- diag(alpha) S + k v^T; o = S^T q.  Returns o [T,H,dv], S [H,d,dv]."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[2], dtype=F64) if S0 is None else S0.clone()
    o = torch.zeros(T, H, v.shape[2], dtype=F64)
    alpha = torch.sigmoid(z) ** (1.0 / tau)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o, S


def polynorm(z, coef, eps):
    a, b, c, e = [float(x) for x in coef]
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


def route(logits, top):
    """indices [T, top] and softmax weights over the chosen logits."""
    tv, ti = torch.topk(logits, top, dim=-1)
    return ti, torch.softmax(tv, -1)


def silu(z):
    return z * torch.sigmoid(z)


class OracleModel:
    """Whole model from a dict of tensors (checkpoint names) and the config dict."""

    def __init__(self, config, tensors):
        self.c = config
        self.w = {k: v.to(F64) for k, v in tensors.items()}
        self.eps = config["norm"]["eps"]

    def mixer(self, i, L, h):
        w, p, m = self.w, f"l{i}.mix.", L["mixer"]
        T = h.shape[0]
        if L["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, d)
            k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, d)
            v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
            o = sliding_sink_attention(q, k, v, m["scale"], m["mask"]["size"], w[p + "sink"], h @ w[p + "g"].T, self.eps)
            return o.reshape(T, H * dv) @ w[p + "o"].T
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        q = (h @ w[p + "q"].T).view(T, H, d) * d ** -0.5
        k = (h @ w[p + "k"].T).view(T, H, d)
        v = (h @ w[p + "v"].T).view(T, H, dv)
        z = ((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]).view(T, H, d)
        o, _ = gla_recurrent(q, k, v, z, m["tau"])
        o = rms_norm(o, w[p + "norm"], self.eps).reshape(T, H * dv) * silu(h @ w[p + "g"].T)
        return o @ w[p + "o"].T

    def feed_forward(self, i, f, h):
        w, p = self.w, f"l{i}.mlp."
        if f["kind"] == "dense":
            return polynorm(h @ w[p + "up"].T, w[p + "act"], self.eps) @ w[p + "down"].T
        ti, tw = route(h @ w[p + "router"].T + w[p + "router.b"], f["router"]["top"])
        out = torch.zeros_like(h)
        for t in range(h.shape[0]):
            for r in range(ti.shape[1]):
                e = int(ti[t, r])
                out[t] += tw[t, r] * ((silu(h[t] @ w[f"{p}e{e}.gate"].T) * (h[t] @ w[f"{p}e{e}.up"].T)) @ w[f"{p}e{e}.down"].T)
        return out

    def forward(self, tokens, taps=None):
        w = self.w
        x = w["embed"][torch.tensor(tokens)] * self.c["embedding"]["scale"]
        for i, L in enumerate(self.c["layers"]):
            h = rms_norm(x, w[f"l{i}.norm1"], self.eps)
            x = x + self.mixer(i, L, h) * torch.sigmoid(h @ w[f"l{i}.rg1"].T + w[f"l{i}.rg1.b"])
            if L["mlp"] is not None:
                h = rms_norm(x, w[f"l{i}.norm2"], self.eps)
                x = x + self.feed_forward(i, L["mlp"], h) * torch.sigmoid(h @ w[f"l{i}.rg2"].T + w[f"l{i}.rg2.b"])
            if taps is not None:
                taps.append(x.clone())
        return rms_norm(x, w["final.norm"], self.eps) @ w["head"].T


def random_model(layers, vocab=96, width=64, seed=0, eps=1e-5, embed_scale=0.7, wscale=1.0):
    """config dict + bfloat16 tensors (checkpoint names) of a small random model.  `layers`: list of dicts
    {"type": "attention", heads, kv_heads, dim, vdim, window, mlp} / {"type": "gla", heads, dim, vdim, tau, rank, mlp};
    mlp: None | ("dense", ff) | ("moe", ff, experts, top)."""
    g = torch.Generator().manual_seed(seed)
    t = {}

    def lin(name, o, i, s=1.0):
        t[name] = (torch.randn(o, i, generator=g) * s * wscale / math.sqrt(i)).to(torch.bfloat16)

    def vec(name, n, mean=0.0, s=0.5):
        t[name] = (mean + torch.randn(n, generator=g) * s).to(torch.bfloat16)
    t["embed"] = torch.randn(vocab, width, generator=g).to(torch.bfloat16)
    lin("head", vocab, width)
    vec("final.norm", width, 1.0, 0.1)
    cl = []
    for i, L in enumerate(layers):
        p = f"l{i}."
        vec(p + "norm1", width, 1.0, 0.1)
        lin(p + "rg1", width, width); vec(p + "rg1.b", width, 0.5)
        if L["type"] == "attention":
            H, G, d, dv = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
            lin(p + "mix.q", H * d, width, 2.0); vec(p + "mix.q.b", H * d)
            lin(p + "mix.k", G * d, width, 2.0); vec(p + "mix.k.b", G * d)
            lin(p + "mix.v", G * dv, width); vec(p + "mix.v.b", G * dv)
            lin(p + "mix.g", H, width); vec(p + "mix.sink", H, 0.0, 1.0)
            lin(p + "mix.o", width, H * dv)
            mixer = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": L.get("scale", d ** -0.5), "mask": {"size": L["window"]}}
        else:
            H, d, dv, r = L["heads"], L["dim"], L["vdim"], L.get("rank", 8)
            lin(p + "mix.q", H * d, width); lin(p + "mix.k", H * d, width); lin(p + "mix.v", H * dv, width); lin(p + "mix.g", H * dv, width)
            lin(p + "mix.a1", r, width); lin(p + "mix.a2", H * d, r, 2.0); vec(p + "mix.a2.b", H * d, L.get("decay_bias", 2.0), 1.0)
            vec(p + "mix.norm", dv, 1.0, 0.1); lin(p + "mix.o", width, H * dv)
            mixer = {"heads": H, "dim": d, "vdim": dv, "tau": L["tau"]}
        f = L.get("mlp")
        if f is None:
            mlp = None
        else:
            vec(p + "norm2", width, 1.0, 0.1)
            lin(p + "rg2", width, width); vec(p + "rg2.b", width, 0.5)
            if f[0] == "dense":
                lin(p + "mlp.up", f[1], width); lin(p + "mlp.down", width, f[1])
                t[p + "mlp.act"] = torch.tensor([0.6, 0.3, -0.2, 0.1]).to(torch.bfloat16)
                mlp = {"kind": "dense", "ff": f[1]}
            else:
                _, ff, E, top = f
                for e in range(E):
                    lin(f"{p}mlp.e{e}.gate", ff, width); lin(f"{p}mlp.e{e}.up", ff, width); lin(f"{p}mlp.e{e}.down", width, ff)
                lin(p + "mlp.router", E, width, 3.0); vec(p + "mlp.router.b", E)
                mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": top}}
        cl.append({"type": L["type"], "mixer": mixer, "mlp": mlp})
    config = {"architecture": "Vofanex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": embed_scale}, "layers": cl}
    return config, t


def save_model(directory, config, tensors):
    import json, os
    from safetensors.torch import save_file
    os.makedirs(directory, exist_ok=True)
    with open(os.path.join(directory, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(directory, "model.safetensors"))

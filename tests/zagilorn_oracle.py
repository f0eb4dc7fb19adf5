"""Slow float64 restatement of the Zagilorn mechanisms, one function per mechanism, written from their equations and sharing no code with
exllamav3_amd (test infrastructure only).  Weights are a dict name -> tensor (used at the stored values), the configuration is the
config.json dict.  Everything runs on the CPU over whole sequences; nothing is cached."""
import math
import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dyn_tanh(x, alpha, w, b):
    """Dynamic Tanh: no statistics of the row at all."""
    return torch.tanh(alpha * x) * w + b


def rotary_tables(positions, dims, base, scaling=None):
    """cos, sin [T, dims/2] for the interleaved pairs (2i, 2i+1); YaRN blends the frequencies and scales both tables."""
    i = torch.arange(dims // 2, dtype=F64)
    f = float(base) ** (-2.0 * i / dims)
    mag = 1.0
    if scaling is not None:
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        where = lambda turns: dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(where(float(scaling["fast"]))), 0)
        hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    a = positions.to(F64)[:, None] * f[None, :]
    return torch.cos(a) * mag, torch.sin(a) * mag


def rotate_pairs(x, cos, sin, dims):
    """x [T, ..., d]: the first `dims` entries of the last axis are rotated pair by pair, the rest pass."""
    out = x.clone()
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = cos.reshape(shape), sin.reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def windowed_softmax_attention(q, k, v, scale, window, sink=None):
    """q, k [T,H,d], v [T,H,dv]; token i sees j with 0 <= i-j < window; the sink (per head) is one more term of the denominator."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        for i in range(T):
            lo = max(0, i - window + 1)
            s = (k[lo:i + 1, h] @ q[i, h]) * scale
            m = s.max() if sink is None else torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink[h] - m) if sink is not None else 0.0)
            out[i, h] = (e / den) @ v[lo:i + 1, h]
    return out


def latent_attention(h, W, pre, m, eps, sink_and_gate, positions=None):
    """One latent-attention mixer over a whole sequence h [T, width].  m = the layer's `mixer` dict."""
    T = h.shape[0]
    H, d, r, dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(T) if positions is None else positions
    q = (h @ W[pre + "q"].T).reshape(T, H, d + r)
    dkv = h @ W[pre + "dkv"].T
    c = unit_rms(dkv[:, :rank], eps) * W[pre + "dkv.norm"]
    k_rot = dkv[:, rank:].reshape(T, 1, r)
    rot = m["rot"]
    dims = int(rot["dims"])
    cos, sin = rotary_tables(pos, dims, rot["base"], rot.get("scaling"))
    q_rot = rotate_pairs(q[:, :, d:], cos, sin, dims)
    k_rot = rotate_pairs(k_rot, cos, sin, dims)
    k_nope = (c @ W[pre + "uk"].T).reshape(T, H, d)
    v = (c @ W[pre + "uv"].T).reshape(T, H, dv)
    qq = torch.cat([q[:, :, :d], q_rot], -1)
    kk = torch.cat([k_nope, k_rot.expand(T, H, r)], -1)
    o = windowed_softmax_attention(qq, kk, v, float(m["scale"]), int(m["mask"]["size"]), W[pre + "sink"] if sink_and_gate else None).reshape(T, H * dv)
    if sink_and_gate:
        o = o * torch.sigmoid(h @ W[pre + "g"].T)
    return o @ W[pre + "o"].T


def relu2_mlp(h, W, pre):
    return torch.relu(h @ W[pre + "up"].T) ** 2 @ W[pre + "down"].T


def clamped_expert(h, W, pre, limit):
    g = torch.clamp(h @ W[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ W[pre + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[pre + "down"].T


def sigmoid_route(z, correction, top, scale):
    """indices [T, top], weights [T, top]: the choice looks at sigmoid(z) + correction, the weights at sigmoid(z) alone."""
    s = torch.sigmoid(z)
    idx = torch.topk(s + correction, top, dim=-1).indices
    w = torch.gather(s, 1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20) * scale


def sparse_mlp(h, W, pre, f):
    idx, wts = sigmoid_route(h @ W[pre + "router"].T, W[pre + "correction"], int(f["router"]["top"]), float(f["router"]["scale"]))
    out = torch.zeros(h.shape[0], W[pre + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            out[t] += wts[t, j] * clamped_expert(h[t:t + 1], W, f"{pre}e{e}.", float(f["expert"]["limit"]))[0]
    if f.get("shared") is not None:
        out = out + clamped_expert(h, W, pre + "shared.", float(f["shared"]["limit"]))
    return out


def token_side(x, tokens, W, pre, layer, dim, eps):
    e = W["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ W[pre + "side.gate"].T) * e) @ W[pre + "side.proj"].T
    return unit_rms(y, eps) * W[pre + "side.norm"]


def layer_forward(x, tokens, W, cfg, i):
    L, eps, pre = cfg["layers"][i], float(cfg["norm"]["eps"]), f"l{i}."
    norm = lambda t, nm: dyn_tanh(t, W[nm + ".alpha"], W[nm], W[nm + ".b"])
    if L["type"] not in ("latent_attention", "latent_attention_2"):
        raise ValueError(L["type"])
    x = x + latent_attention(norm(x, pre + "norm1"), W, pre + "mix.", L["mixer"], eps, L["type"] == "latent_attention")
    f = L.get("mlp")
    if f is not None:
        hh = norm(x, pre + "norm2")
        x = x + (relu2_mlp(hh, W, pre + "mlp.") if f["kind"] == "dense" else sparse_mlp(hh, W, pre + "mlp.", f))
    if cfg.get("token_side") is not None:
        x = x + token_side(x, tokens, W, pre, i, int(cfg["token_side"]["dim"]), eps)
    return x


def layer_runs(cfg):
    """The order in which layers run: (layer, first of a pass?) with the looped block repeated."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if loop is None:
        return [(i, False) for i in range(n)]
    a, b, t = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for _ in range(t):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(tokens, weights, cfg, taps=None):
    """Logits [T, vocab] of one whole sequence; taps (a list) receives the residual after every layer run."""
    W = {k: v.to(F64) for k, v in weights.items() if v.dtype != torch.int32}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x0 = W["embed"][tokens]
    x = x0
    for i, inject in layer_runs(cfg):
        if inject:
            x = torch.cat([x, x0], -1) @ W["loop.in"].T
        x = layer_forward(x, tokens, W, cfg, i)
        if taps is not None:
            taps.append(x.clone())
    h = dyn_tanh(x, W["final.norm.alpha"], W["final.norm"], W["final.norm.b"])
    return (h @ W["head"].T) * float(cfg.get("logit_scale", 1.0))


def greedy(prompt, n_new, weights, cfg):
    toks, out = list(prompt), []
    for _ in range(n_new):
        t = int(forward(toks, weights, cfg)[-1].argmax())
        out.append(t); toks.append(t)
    return out

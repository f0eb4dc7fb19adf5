"""
Zagilorn: a decoder-only model of pre-norm blocks over a float32 stream -- latent attention (a cached low-rank latent and one shared rotated key
part per token, rotary positions, sliding window; with or without sink, output gate and YaRN), a relu^2 feed-forward or sigmoid-routed clamped
experts with a shared expert, and a per-layer token input from a second embedding -- normed by Dynamic Tanh.  A block of consecutive layers may
run several times in a row with the same weights; each pass has its own cache, and each pass starts from a linear map of [stream | embedding].
The order of layers and every size and constant come from config.json:

    architecture "Zagilorn"; vocab; width; norm.eps; logit_scale; token_side.dim (optional); loop {start, stop, times} (optional)
    layers[i]: type ("latent_attention": sink, gate | "latent_attention_2": neither), mixer {heads, dim, rot_dim, vdim, kv_rank, scale, mask.size,
               rot {base, dims, scaling {factor, original, fast, slow} (optional)}},
               mlp ({"kind": "dense", "ff"} | {"kind": "moe", "expert": {ff, limit}, "router": {experts, top, scale}, "shared": {ff, limit} (optional)} | null)

Tensor names: embed, head, final.norm(.b, .alpha), loop.in, side.embed, l<i>.norm1 / norm2 (.b, .alpha), l<i>.mix.*, l<i>.mlp.*, l<i>.side.*.

The model is a list of PreNormBlock over the mechanisms of modules.py; its state is a SlotStateCache with one entry per layer RUN (a looped layer has one
ring per pass); `step` is the one function the generator, the command line and the trace runner call.
"""
from __future__ import annotations
import json
import os
import torch
import torch.nn.functional as F
from . import mix_ops
from .loader import SafetensorsCollection
from .modules import ActMLP, DynTanh, GatedMLP, LatentAttention, NextInput, PreNormBlock, SparseExperts, TokenSide, update_residual, _w
from .state_cache import SlotStateCache, StepBatch

MIXER_TYPES = {"latent_attention": dict(sink=True, gate=True), "latent_attention_2": dict(sink=False, gate=False)}


class ZagilornConfig:
    def __init__(self, d: dict):
        self.vocab = int(d["vocab"])
        self.width = int(d["width"])
        self.eps = float(d["norm"]["eps"])
        self.logit_scale = float(d.get("logit_scale", 1.0))
        self.layers = d["layers"]
        if not self.layers:
            raise RuntimeError("Zagilorn: config has no layers")
        ts = d.get("token_side")
        self.side_dim = int(ts["dim"]) if ts else 0
        loop = d.get("loop")
        n = len(self.layers)
        if loop:
            self.loop = (int(loop["start"]), int(loop["stop"]), int(loop["times"]))
            a, b, t = self.loop
            if not (0 <= a < b <= n and t >= 1):
                raise RuntimeError(f"Zagilorn: loop {self.loop} does not fit {n} layers")
        else:
            self.loop = None

    def runs(self) -> list[tuple[int, bool]]:
        """(layer, starts a pass of the loop) in execution order."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        a, b, t = self.loop
        out = [(i, False) for i in range(a)]
        for _ in range(t):
            out += [(i, i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, n)]

    def build_layers(self) -> list[PreNormBlock]:
        out = []
        for i, L in enumerate(self.layers):
            if L["type"] not in MIXER_TYPES:
                raise RuntimeError(f"Zagilorn: layer {i} has an unknown mixer type {L['type']!r}")
            m, rot = L["mixer"], L["mixer"]["rot"]
            mixer = LatentAttention(self.width, int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]), float(m["scale"]),
                                    int(m["mask"]["size"]), self.eps, int(rot.get("dims", m["rot_dim"])), float(rot["base"]), rot.get("scaling"), **MIXER_TYPES[L["type"]])
            f = L.get("mlp")
            if f is None:
                mlp = None
            elif f["kind"] == "dense":
                mlp = ActMLP(self.width, int(f["ff"]), "relu2")
            elif f["kind"] == "moe":
                sh = f.get("shared")
                shared = GatedMLP(self.width, int(sh["ff"]), "clamped_swish", float(sh["limit"])) if sh else None
                mlp = SparseExperts(self.width, int(f["expert"]["ff"]), int(f["router"]["experts"]), int(f["router"]["top"]), router="sigmoid", router_bias=False,
                                    correction=True, route_scale=float(f["router"].get("scale", 1.0)), act="clamped_swish", limit=float(f["expert"]["limit"]), shared=shared)
            else:
                raise RuntimeError(f"Zagilorn: layer {i} has an unknown feed-forward kind {f['kind']!r}")
            side = TokenSide(self.width, self.side_dim, i, self.eps) if self.side_dim else None
            out.append(PreNormBlock(self.width, self.eps, mixer, mlp, side))
        return out


class ZagilornModel:
    architecture = "Zagilorn"
    native_libraries = ("mix",)          # what a fresh checkout has to compile before this model runs

    def __init__(self, config: dict, stc, device="cuda:0", dtype=torch.bfloat16):
        if dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError("Zagilorn runs in bfloat16 or float32")
        self.cfg = ZagilornConfig(config)
        self.device, self.dtype = torch.device(device), dtype
        self.vocab = self.cfg.vocab
        self.blocks = self.cfg.build_layers()
        self.side_table = _w(stc, "side.embed", dtype, self.device) if self.cfg.side_dim else None
        for i, blk in enumerate(self.blocks):
            blk.load(stc, f"l{i}.", dtype, self.device, self.side_table)
        self.runs = self.cfg.runs()
        self.embed = _w(stc, "embed", dtype, self.device)
        self.head = _w(stc, "head", dtype, self.device)
        self.final_norm = DynTanh(self.cfg.width).load(stc, "final.norm", self.device)
        self.loop_in = _w(stc, "loop.in", dtype, self.device) if self.cfg.loop else None
        w = self.cfg.width
        assert self.embed.shape == (self.vocab, w) and self.head.shape == (self.vocab, w)
        assert self.loop_in is None or self.loop_in.shape == (w, 2 * w)
        assert self.side_table is None or self.side_table.shape == (self.vocab, len(self.blocks) * self.cfg.side_dim)
        self.layer_taps = None               # diagnostics: a list that receives a copy of the residual after every layer run

    @classmethod
    def from_directory(cls, directory: str, device="cuda:0", dtype=torch.bfloat16) -> "ZagilornModel":
        with open(os.path.join(directory, "config.json")) as f:
            config = json.load(f)
        return cls(config, SafetensorsCollection(directory), device=device, dtype=dtype)

    def new_cache(self, slots: int = 4) -> SlotStateCache:
        """One state entry per layer run: a layer inside the loop holds one ring per pass."""
        return SlotStateCache([self.blocks[i].state_specs() for i, _ in self.runs], self.device, slots=slots)

    @torch.no_grad()
    def step(self, sb: StepBatch, cache: SlotStateCache) -> torch.Tensor | None:
        """Run the step's rows through every layer run over the slots of `cache`; returns float32 logits [wanted rows, vocab] (None if none are wanted)."""
        w, n = self.cfg.width, sb.n
        x = torch.empty((n, w), dtype=torch.float32, device=self.device)
        # a pass of the loop reads [stream | embedding]: the right half is written once, the left half by whichever update precedes a pass
        both = torch.empty((n, 2 * w), dtype=self.dtype, device=self.device) if self.loop_in is not None else None
        left = both[:, :w] if both is not None else None
        mix_ops.embed_copy(x, both[:, w:] if both is not None else None, self.embed, sb.tokens)
        h = torch.empty((n, w), dtype=self.dtype, device=self.device)
        first_layer, first_injects = self.runs[0]
        if first_injects:
            update_residual(x, None, NextInput(None, left), mode=mix_ops.RES_KEEP)
        else:
            update_residual(x, None, NextInput(self.blocks[first_layer].norm1, h), mode=mix_ops.RES_KEEP)
        for r, (i, injects) in enumerate(self.runs):
            blk = self.blocks[i]
            if injects:
                update_residual(x, F.linear(both, self.loop_in), NextInput(blk.norm1, h), mode=mix_ops.RES_SET)
            if r + 1 == len(self.runs):
                nxt = None
            elif self.runs[r + 1][1]:
                nxt = NextInput(None, left)
            else:
                h_next = torch.empty((n, w), dtype=self.dtype, device=self.device)
                nxt = NextInput(self.blocks[self.runs[r + 1][0]].norm1, h_next)
            blk.forward(x, h, sb, cache.layers[r], nxt)
            if nxt is not None and nxt.norm is not None:
                h = nxt.out
            if self.layer_taps is not None:
                self.layer_taps.append(x.clone())
        if sb.want_rows is None or sb.want_rows.numel() == 0:
            return None
        hw = torch.empty((sb.want_rows.numel(), w), dtype=self.dtype, device=self.device)
        mix_ops.dyn_tanh_rows(hw, x, sb.want_rows, self.final_norm.alpha, self.final_norm.w, self.final_norm.b)
        logits = F.linear(hw, self.head).float()
        return logits * self.cfg.logit_scale if self.cfg.logit_scale != 1.0 else logits

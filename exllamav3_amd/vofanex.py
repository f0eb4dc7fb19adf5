"""
Vofanex: a decoder-only model whose layers pair a sequence mixer -- sliding-window attention with a sink, or gated linear attention --
with a PolyNorm feed-forward, a sparse mixture of experts, or none, every sublayer behind a sigmoid-gated residual over a float32
stream.  The order of layers and every size and constant come from config.json:

    architecture "Vofanex"; vocab; width; norm.eps; embedding.scale;
    layers[i]: type ("attention" | "gla"), mixer {...}, mlp ({"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}} | null)
      attention mixer: heads, kv_heads, dim, vdim, scale, mask.size        gla mixer: heads, dim, vdim, tau

Tensor names: embed, head, final.norm, l<i>.norm1 / norm2 / rg1(.b) / rg2(.b), l<i>.mix.*, l<i>.mlp.* (modules.py reads them).

The model is a list of GatedResidualBlock over the mechanisms of modules.py; its state is a SlotStateCache; `step` is the one function
the generator, the command line and the trace runner call.
"""
from __future__ import annotations
import json
import os
import torch
import torch.nn.functional as F
from . import mix_ops
from .loader import SafetensorsCollection
from .modules import GatedLinearAttention, GatedResidualBlock, PolyNormMLP, SlidingSinkAttention, SparseExperts, _f32, _w
from .state_cache import SlotStateCache, StepBatch


class VofanexConfig:
    def __init__(self, d: dict):
        self.vocab = int(d["vocab"])
        self.width = int(d["width"])
        self.eps = float(d["norm"]["eps"])
        self.embed_scale = float(d.get("embedding", {}).get("scale", 1.0))
        self.layers = d["layers"]
        if not self.layers:
            raise RuntimeError("Vofanex: config has no layers")

    def build_layers(self) -> list[GatedResidualBlock]:
        out = []
        for i, L in enumerate(self.layers):
            m = L["mixer"]
            if L["type"] == "attention":
                mixer = SlidingSinkAttention(self.width, int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                                             float(m["scale"]), int(m["mask"]["size"]), self.eps)
            elif L["type"] == "gla":
                mixer = GatedLinearAttention(self.width, int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])), float(m["tau"]), self.eps)
            else:
                raise RuntimeError(f"Vofanex: layer {i} has an unknown mixer type {L['type']!r}")
            f = L.get("mlp")
            if f is None:
                mlp = None
            elif f["kind"] == "dense":
                mlp = PolyNormMLP(self.width, int(f["ff"]), self.eps)
            elif f["kind"] == "moe":
                mlp = SparseExperts(self.width, int(f["expert"]["ff"]), int(f["router"]["experts"]), int(f["router"]["top"]))
            else:
                raise RuntimeError(f"Vofanex: layer {i} has an unknown feed-forward kind {f['kind']!r}")
            out.append(GatedResidualBlock(self.width, self.eps, mixer, mlp))
        return out


class VofanexModel:
    architecture = "Vofanex"
    native_libraries = ("mix",)          # what a fresh checkout has to compile before this model runs

    def __init__(self, config: dict, stc, device="cuda:0", dtype=torch.bfloat16):
        if dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError("Vofanex runs in bfloat16 or float32")
        self.cfg = VofanexConfig(config)
        self.device, self.dtype = torch.device(device), dtype
        self.vocab = self.cfg.vocab
        self.blocks = self.cfg.build_layers()
        for i, blk in enumerate(self.blocks):
            blk.load(stc, f"l{i}.", dtype, self.device)
        self.embed = _w(stc, "embed", dtype, self.device)
        self.head = _w(stc, "head", dtype, self.device)
        self.final_norm = _f32(stc, "final.norm", self.device)
        assert self.embed.shape == (self.vocab, self.cfg.width) and self.head.shape == (self.vocab, self.cfg.width)
        self.layer_taps = None               # diagnostics: a list that receives a copy of the residual after every layer

    @classmethod
    def from_directory(cls, directory: str, device="cuda:0", dtype=torch.bfloat16) -> "VofanexModel":
        with open(os.path.join(directory, "config.json")) as f:
            config = json.load(f)
        return cls(config, SafetensorsCollection(directory), device=device, dtype=dtype)

    def new_cache(self, slots: int = 4) -> SlotStateCache:
        return SlotStateCache([b.state_specs() for b in self.blocks], self.device, slots=slots)

    @torch.no_grad()
    def step(self, sb: StepBatch, cache: SlotStateCache) -> torch.Tensor | None:
        """Run the step's rows through every layer over the slots of `cache`; returns float32 logits [wanted rows, vocab] (None if none are wanted)."""
        w = self.cfg.width
        x = torch.empty((sb.n, w), dtype=torch.float32, device=self.device)
        h = torch.empty((sb.n, w), dtype=self.dtype, device=self.device)
        mix_ops.embed(x, h, self.embed, sb.tokens, self.cfg.embed_scale, self.blocks[0].norm1, self.cfg.eps)
        for i, blk in enumerate(self.blocks):
            nxt = self.blocks[i + 1].norm1 if i + 1 < len(self.blocks) else None
            h = blk.forward(x, h, sb, cache.layers[i], nxt)
            if self.layer_taps is not None:
                self.layer_taps.append(x.clone())
        if sb.want_rows is None or sb.want_rows.numel() == 0:
            return None
        hw = torch.empty((sb.want_rows.numel(), w), dtype=self.dtype, device=self.device)
        mix_ops.rms_norm_rows(hw, x, sb.want_rows, self.final_norm, self.cfg.eps)
        return F.linear(hw, self.head).float()

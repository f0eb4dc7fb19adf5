"""
Building blocks of the unquantized mixer models: each mechanism is one class with its constants as constructor arguments, its tensors
read through the framework's SafetensorsCollection, its per-slot state declared as StateSpec, and a forward over a packed StepBatch that
runs the kernels of libexl3_mix.so (mix_ops) around vendor matrix products (torch.nn.functional.linear: hipBLASLt / rocBLAS with
float32 accumulation; true float32 when the model runs in float32).

    FusedInput              several linears over one input as one matrix product, outputs as column views
    SlidingSinkAttention    grouped-query attention over a sliding window, optional learned sink in the softmax denominator, optional unit-RMS
                            values, optional head-wise sigmoid output gate, no rotation; ring cache of `window` entries per slot
    GatedLinearAttention    linear attention with a low-rank per-channel decay sigmoid(z)^(1/tau), float32 state per head, per-head RMS norm,
                            silu output gate
    PolyNormMLP             W_down act(W_up h), act = a N(z) + b N(z^2) + c N(z^3) + e
    SparseExperts           top-k of n experts (router in float32, softmax over the chosen logits), experts W_down (silu(W_gate h) * W_up h)
    GatedResidualBlock      x += sublayer(norm(x)) * sigmoid(W norm(x) + b) for a mixer and an optional feed-forward, residual in float32

Every sum that the model's exactness rests on (norms, scores, softmax, decays, states, the residual) is float32 inside the kernels in
both modes; the element type only decides how matrix products and their outputs are held.
"""
from __future__ import annotations
import torch
import torch.nn.functional as F
from . import mix_ops
from .state_cache import StateSpec, StepBatch


def _w(stc, key: str, dtype, device) -> torch.Tensor:
    return stc.get_tensor(key, device="cpu").to(dtype).to(device).contiguous()


def _f32(stc, key: str, device) -> torch.Tensor:
    return stc.get_tensor(key, device="cpu").to(torch.float32).to(device).contiguous()


class FusedInput:
    """Linears that read the same input, stacked into one weight: one matrix product instead of several, and every consumer kernel takes its
    column block in place (row stride = total width).  Parts without a bias get zeros in the fused bias (adding zero is exact)."""

    def __init__(self, parts: list[tuple[str, torch.Tensor, torch.Tensor | None]]):
        self.names = [p[0] for p in parts]
        self.sizes = [p[1].shape[0] for p in parts]
        self.weight = torch.cat([p[1] for p in parts], dim=0).contiguous()
        if any(p[2] is not None for p in parts):
            self.bias = torch.cat([p[2].to(self.weight.dtype) if p[2] is not None else torch.zeros(p[1].shape[0], dtype=self.weight.dtype, device=self.weight.device)
                                   for p in parts]).contiguous()
        else:
            self.bias = None
        self.offsets, at = {}, 0
        for n, s in zip(self.names, self.sizes):
            self.offsets[n] = (at, s); at += s

    def __call__(self, h: torch.Tensor) -> dict[str, torch.Tensor]:
        out = F.linear(h, self.weight, self.bias)
        return {n: out[:, a: a + s] for n, (a, s) in self.offsets.items()}


class SlidingSinkAttention:
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, window: int, eps: float, sink: bool = True,
                 value_norm: bool = True, gate: bool = True, bias: bool = True):
        if heads % kv_heads:
            raise RuntimeError(f"attention: {heads} query heads over {kv_heads} key/value heads")
        if not value_norm:
            raise RuntimeError("attention: the cache store kernel normalises values; an un-normalised variant is not built")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim = width, heads, kv_heads, dim, vdim
        self.scale, self.window, self.eps = float(scale), int(window), float(eps)
        self.has_sink, self.has_gate, self.has_bias = sink, gate, bias

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        parts = []
        for nm in ("q", "k", "v"):
            parts.append((nm, _w(stc, prefix + nm, dtype, device), _w(stc, prefix + nm + ".b", dtype, device) if self.has_bias else None))
        if self.has_gate:
            parts.append(("g", _w(stc, prefix + "g", dtype, device), None))
        self.inp = FusedInput(parts + list(extra_parts))
        self.sink = _f32(stc, prefix + "sink", device) if self.has_sink else None
        self.w_o = _w(stc, prefix + "o", dtype, device)
        assert self.inp.offsets["q"][1] == self.heads * self.dim and self.inp.offsets["v"][1] == self.kv_heads * self.vdim
        assert self.w_o.shape == (self.width, self.heads * self.vdim)
        self.dtype = dtype

    def state_specs(self) -> list[StateSpec]:
        return [StateSpec("ring_k", (self.window, self.kv_heads, self.dim), self.dtype), StateSpec("ring_v", (self.window, self.kv_heads, self.vdim), self.dtype)]

    def forward(self, h: torch.Tensor, sb: StepBatch, state: dict) -> tuple[torch.Tensor, dict]:
        p = self.inp(h)
        v_norm = torch.empty((sb.n, self.kv_heads, self.vdim), dtype=self.dtype, device=h.device)
        mix_ops.attn_store(v_norm, state["ring_k"], state["ring_v"], p["k"], p["v"], sb.tok_seq, sb.tok_pos, sb.slots, sb.len_after, self.eps)
        out = torch.empty((sb.n, self.heads * self.vdim), dtype=self.dtype, device=h.device)
        if sb.decode:
            mix_ops.attn_decode(out, p["q"], state["ring_k"], state["ring_v"], p.get("g"), self.sink, sb.slots, sb.len_after, self.heads, self.scale)
        else:
            mix_ops.attn_prefill(out, p["q"], p["k"], v_norm, p.get("g"), self.sink, sb.cu, sb.tok_seq, sb.tok_pos, self.heads, self.scale, self.window,
                                 max_rows=sb.max_rows)
        return F.linear(out, self.w_o), p


class GatedLinearAttention:
    # prompt steps whose longest sequence has at least this many rows are cut into parallel time segments (mix_ops.gla_scan)
    SEGMENT_MIN_ROWS = 256
    SEGMENT_TARGET_WORKGROUPS = 1024

    def __init__(self, width: int, heads: int, dim: int, vdim: int, tau: float, eps: float):
        self.width, self.heads, self.dim, self.vdim, self.tau, self.eps = width, heads, dim, vdim, float(tau), float(eps)
        self.q_scale = float(dim) ** -0.5

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        parts = [(nm, _w(stc, prefix + nm, dtype, device), None) for nm in ("q", "k", "v", "g", "a1")]
        self.inp = FusedInput(parts + list(extra_parts))
        self.a2 = _w(stc, prefix + "a2", dtype, device)
        self.a2_bias = _f32(stc, prefix + "a2.b", device)
        self.norm_w = _f32(stc, prefix + "norm", device)
        self.w_o = _w(stc, prefix + "o", dtype, device)
        assert self.inp.offsets["q"][1] == self.heads * self.dim and self.inp.offsets["v"][1] == self.heads * self.vdim
        assert self.a2.shape[0] == self.heads * self.dim and self.a2.shape[1] == self.inp.offsets["a1"][1]
        self.dtype = dtype

    def state_specs(self) -> list[StateSpec]:
        return [StateSpec("S", (self.heads, self.dim, self.vdim), torch.float32)]

    def segments(self, sb: StepBatch) -> tuple[int, int] | None:
        """(segments per sequence, rows per segment) for a long prompt step: enough workgroups to fill the device, segments of at least 64 rows."""
        if sb.max_rows < self.SEGMENT_MIN_ROWS:
            return None
        chains = sb.batch * self.heads * ((self.vdim + 63) // 64)
        segs = min(max(1, -(-self.SEGMENT_TARGET_WORKGROUPS // chains)), sb.max_rows // 64)
        if segs < 2:
            return None
        seg_len = -(-sb.max_rows // segs)
        seg_len = -(-seg_len // 16) * 16
        return -(-sb.max_rows // seg_len), seg_len

    def forward(self, h: torch.Tensor, sb: StepBatch, state: dict) -> tuple[torch.Tensor, dict]:
        p = self.inp(h)
        o = torch.empty((sb.n, self.heads, self.vdim), dtype=torch.float32, device=h.device)
        mix_ops.gla_scan(o, state["S"], p["q"], p["k"], p["v"], p["a1"], self.a2, self.a2_bias, sb.cu, sb.slots, sb.pos0, self.tau, self.q_scale,
                         segments=self.segments(sb))
        out = torch.empty((sb.n, self.heads * self.vdim), dtype=self.dtype, device=h.device)
        mix_ops.gla_out(out, o, self.norm_w, p["g"], self.eps)
        return F.linear(out, self.w_o), p


class PolyNormMLP:
    def __init__(self, width: int, ff: int, eps: float):
        self.width, self.ff, self.eps = width, ff, float(eps)

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        self.inp = FusedInput([("up", _w(stc, prefix + "up", dtype, device), None)] + list(extra_parts))
        self.coef = _f32(stc, prefix + "act", device)
        self.w_down = _w(stc, prefix + "down", dtype, device)
        assert self.inp.offsets["up"][1] == self.ff and self.w_down.shape == (self.width, self.ff)
        self.dtype = dtype

    def forward(self, h: torch.Tensor, sb: StepBatch) -> tuple[torch.Tensor, dict]:
        p = self.inp(h)
        a = torch.empty((sb.n, self.ff), dtype=self.dtype, device=h.device)
        mix_ops.polynorm(a, p["up"], self.coef, self.eps)
        return F.linear(a, self.w_down), p


class SparseExperts:
    # rows from which the expert-sorted matrix products take over from the weight-streaming kernels, and rows from which the streaming kernels
    # walk each chosen expert once for all its rows instead of once per (row, choice)
    GROUPED_MIN_ROWS = 64
    EXPERT_MAJOR_MIN_ROWS = 4

    def __init__(self, width: int, ff: int, experts: int, top: int):
        if not 0 < top <= experts:
            raise RuntimeError(f"router: top {top} of {experts} experts")
        self.width, self.ff, self.experts, self.top = width, ff, experts, top

    def load(self, stc, prefix: str, dtype, device, extra_parts=()):
        stack = lambda nm: torch.stack([_w(stc, f"{prefix}e{e}.{nm}", dtype, device) for e in range(self.experts)]).contiguous()
        self.w_gate, self.w_up, self.w_down = stack("gate"), stack("up"), stack("down")
        self.w_router = _f32(stc, prefix + "router", device)
        self.b_router = _f32(stc, prefix + "router.b", device)
        self.inp = FusedInput(list(extra_parts)) if extra_parts else None
        assert self.w_gate.shape == (self.experts, self.ff, self.width) and self.w_down.shape == (self.experts, self.width, self.ff)
        self.dtype = dtype

    def forward(self, h: torch.Tensor, sb: StepBatch) -> tuple[torch.Tensor, dict]:
        p = self.inp(h) if self.inp is not None else {}
        logits = torch.addmm(self.b_router, h.float(), self.w_router.t())          # float32 product of the (rounded) input
        idx = torch.empty((sb.n, self.top), dtype=torch.int32, device=h.device)
        wts = torch.empty((sb.n, self.top), dtype=torch.float32, device=h.device)
        mix_ops.topk_softmax(idx, wts, logits)
        y = torch.empty((sb.n, self.width), dtype=self.dtype, device=h.device)
        if sb.n >= self.GROUPED_MIN_ROWS:
            mix_ops.moe_grouped(y, h, self.w_gate, self.w_up, self.w_down, idx, wts)
        elif sb.n >= self.EXPERT_MAJOR_MIN_ROWS and mix_ops.moe_vector_layout(h, self.ff):
            mix_ops.moe_expert_major(y, h, self.w_gate, self.w_up, self.w_down, idx, wts)
        else:
            hid = torch.empty((sb.n * self.top, self.ff), dtype=self.dtype, device=h.device)
            mix_ops.moe_gate_up(hid, h, self.w_gate, self.w_up, idx)
            mix_ops.moe_down(y, hid, self.w_down, idx, wts)
        return y, p


class GatedResidualBlock:
    """One layer: x <- x + mixer(n1(x)) * sigmoid(W1 n1(x) + b1); x <- x + ff(n2(x)) * sigmoid(W2 n2(x) + b2) (the second half only with a
    feed-forward).  The gate's linear rides in the sublayer's fused input product; the residual add, the gate and the NEXT norm are one kernel."""

    def __init__(self, width: int, eps: float, mixer, mlp):
        self.width, self.eps, self.mixer, self.mlp = width, float(eps), mixer, mlp

    def load(self, stc, prefix: str, dtype, device):
        self.norm1 = _f32(stc, prefix + "norm1", device)
        self.mixer.load(stc, prefix + "mix.", dtype, device, extra_parts=[("rg", _w(stc, prefix + "rg1", dtype, device), _w(stc, prefix + "rg1.b", dtype, device))])
        if self.mlp is not None:
            self.norm2 = _f32(stc, prefix + "norm2", device)
            self.mlp.load(stc, prefix + "mlp.", dtype, device, extra_parts=[("rg", _w(stc, prefix + "rg2", dtype, device), _w(stc, prefix + "rg2.b", dtype, device))])

    def state_specs(self) -> list[StateSpec]:
        return self.mixer.state_specs()

    def forward(self, x: torch.Tensor, h: torch.Tensor, sb: StepBatch, state: dict, next_norm: torch.Tensor | None) -> torch.Tensor | None:
        """x: float32 residual (updated in place); h = norm1(x) in the activation type.  Returns the next layer's h (None when next_norm is None)."""
        y, p = self.mixer.forward(h, sb, state)
        after = self.norm2 if self.mlp is not None else next_norm
        h2 = torch.empty_like(h) if after is not None else None
        mix_ops.gated_residual(x, y, p["rg"], after, h2, self.eps)
        if self.mlp is None:
            return h2
        y, p = self.mlp.forward(h2, sb)
        h3 = torch.empty_like(h) if next_norm is not None else None
        mix_ops.gated_residual(x, y, p["rg"], next_norm, h3, self.eps)
        return h3

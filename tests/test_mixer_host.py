"""CPU tests of the mixer family's host side: the oracle against closed forms, the slot state manager, the scheduler and sampler over a
stand-in model, the registry and configuration reader, and the C-ABI of libexl3_mix.so (cross-compiled; no GPU)."""
import json
import os
import pytest
import torch
import mixer_oracle as mo

F64 = torch.float64


def test_oracle_gla_equals_the_unrolled_sum():
    g = torch.Generator().manual_seed(0)
    T, H, d, dv = 9, 2, 3, 4
    q, k, z = (torch.randn(T, H, d, generator=g, dtype=F64) for _ in range(3)); v = torch.randn(T, H, dv, generator=g, dtype=F64)
    o, S = mo.gla_recurrent(q, k, v, z, 2.5)
    la = torch.log(torch.sigmoid(z)) / 2.5
    for t in range(T):
        ref = torch.zeros(H, dv, dtype=F64)
        for j in range(t + 1):
            w = torch.exp(la[j + 1: t + 1].sum(0))                 # decays applied after key j was written
            ref += ((q[t] * w * k[j]).sum(-1))[:, None] * v[j]
        assert torch.allclose(o[t], ref, atol=1e-12)


def test_oracle_attention_equals_dense_masked_softmax_with_a_sink_column():
    g = torch.Generator().manual_seed(1)
    T, H, G, d, dv, W = 11, 4, 2, 5, 6, 4
    q = torch.randn(T, H, d, generator=g, dtype=F64); k = torch.randn(T, G, d, generator=g, dtype=F64); v = torch.randn(T, G, dv, generator=g, dtype=F64)
    sink = torch.randn(H, generator=g, dtype=F64)
    got = mo.sliding_sink_attention(q, k, v, 0.4, W, sink, None, 1e-5)
    vn = mo.unit_rms(v, 1e-5)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    mask = (i >= j) & (i - j < W)
    for h in range(H):
        s = (q[:, h] @ k[:, h // 2].T) * 0.4
        s = torch.cat([s.masked_fill(~mask, float("-inf")), sink[h].expand(T, 1)], 1)
        p = torch.softmax(s, -1)[:, :T]
        assert torch.allclose(got[:, h], p @ vn[:, h // 2], atol=1e-12)


def test_slot_cache_hands_out_reuses_and_grows_without_losing_state():
    from exllamav3_amd.state_cache import SlotStateCache, StateSpec
    c = SlotStateCache([[StateSpec("S", (2, 3), torch.float32)], [StateSpec("ring_k", (4, 1, 2), torch.bfloat16)]], "cpu", slots=2)
    a, b = c.alloc(), c.alloc()
    assert (a, b) == (0, 1) and c.in_use() == 2
    c.layers[0]["S"][b].fill_(7.0)
    d = c.alloc()                                                 # pool doubles; slot 1 keeps its contents
    assert d == 2 and c.capacity == 4 and float(c.layers[0]["S"][b].min()) == 7.0
    c.release(a)
    assert c.alloc() == a                                         # the slot given back last is used again first
    with pytest.raises(RuntimeError):
        c.release(3)
    assert c.bytes_per_slot() == 2 * 3 * 4 + 4 * 2 * 2


def test_begin_step_layout_and_rules():
    from exllamav3_amd.state_cache import SlotStateCache, StateSpec
    c = SlotStateCache([[StateSpec("S", (1,), torch.float32)]], "cpu", slots=4)
    s0, s1, s2 = c.alloc(), c.alloc(), c.alloc()
    sb = c.begin_step([(s2, [5, 6, 7]), (s0, [9])], [[0, 2], []])
    assert not sb.decode and sb.n == 4 and sb.batch == 2 and sb.max_rows == 3
    assert sb.cu.tolist() == [0, 3, 4] and sb.tok_seq.tolist() == [0, 0, 0, 1] and sb.tok_pos.tolist() == [0, 1, 2, 0]
    assert sb.slots.tolist() == [s2, s0] and sb.pos0.tolist() == [0, 0] and sb.len_after.tolist() == [3, 1] and sb.want_rows.tolist() == [0, 2]
    sb = c.begin_step([(s0, [1]), (s2, [2])])
    assert sb.decode and sb.tok_pos.tolist() == [1, 3] and sb.want_rows.tolist() == [0, 1] and sb.len_after.tolist() == [2, 4]
    sb = c.begin_step([(s1, [4]), (s0, [3])], [[], []])           # a sequence's first token beside a running one: one token each
    assert sb.decode and sb.pos0.tolist() == [0, 2] and sb.want_rows.numel() == 0
    with pytest.raises(RuntimeError):
        c.begin_step([(s0, [1, 2])])
    with pytest.raises(RuntimeError):
        c.begin_step([(s0, [])])


class CountingModel:
    """Stand-in with the step interface: the next token is (sum of the sequence's tokens so far + its length) mod vocab, kept per slot."""
    vocab, device = 17, torch.device("cpu")

    def __init__(self):
        self.sums, self.steps = {}, []

    def new_cache(self, slots=2):
        from exllamav3_amd.state_cache import SlotStateCache, StateSpec
        return SlotStateCache([[StateSpec("S", (1,), torch.float32)]], "cpu", slots=slots)

    def step(self, sb, cache):
        self.steps.append((sb.decode, sb.slots.tolist(), sb.host_lens))
        out = torch.zeros(sb.batch, self.vocab)
        cu = sb.cu.tolist()
        for i, sl in enumerate(sb.slots.tolist()):
            if sb.pos0[i] == 0:
                self.sums[sl] = 0
            self.sums[sl] += int(sb.tokens[cu[i]: cu[i + 1]].sum())
            out[i, (self.sums[sl] + int(sb.len_after[i])) % self.vocab] = 5.0
        return out


def expected_counting(prompt, new, vocab=17):
    s, out = list(prompt), []
    for _ in range(new):
        out.append((sum(s) + len(s)) % vocab); s.append(out[-1])
    return out


def test_scheduler_batches_admits_into_freed_slots_and_stops():
    from exllamav3_amd.generator import Generator, Job, SamplerSettings
    m = CountingModel()
    gen = Generator(m, max_batch=2, max_step_rows=6)
    prompts = [[1, 2, 3], [4], [5, 6, 7, 8], [9, 9]]
    lens = [3, 6, 2, 4]
    jobs = [gen.enqueue(Job(p, n)) for p, n in zip(prompts, lens)]
    while gen.busy():
        gen.iterate()
    for j, p, n in zip(jobs, prompts, lens):
        assert j.output == expected_counting(p, n) and j.slot is None
    assert gen.cache.in_use() == 0 and gen.cache.capacity == 2    # never more than two alive: no growth, slots were used again
    assert m.steps[0] == (False, [0, 1], [3, 1])                   # first two prompts as one packed step
    assert any(d and len(s) == 2 for d, s, _ in m.steps)          # decoded together
    # stop token ends a job early
    j = gen.enqueue(Job([1, 2, 3], 50, stop_tokens=(expected_counting([1, 2, 3], 3)[-1],)))
    while gen.busy():
        gen.iterate()
    assert j.output == expected_counting([1, 2, 3], 3)
    with pytest.raises(RuntimeError):
        gen.enqueue(Job([99], 1))


def test_sampler_is_greedy_at_zero_temperature_and_reproducible_otherwise():
    from exllamav3_amd.generator import Sampler, SamplerSettings
    l = torch.tensor([0.1, 2.0, -1.0, 1.9, 0.0])
    assert Sampler(SamplerSettings(), "cpu").sample(l) == 1
    assert Sampler(SamplerSettings(temperature=1.0, top_k=1, seed=3), "cpu").sample(l) == 1
    a = [Sampler(SamplerSettings(temperature=1.5, seed=11), "cpu").sample(l) for _ in range(3)]
    assert a[0] == a[1] == a[2]
    s = Sampler(SamplerSettings(temperature=1.0, top_p=0.6, seed=0), "cpu")
    assert {s.sample(l) for _ in range(50)} <= {1, 3}            # the two tokens that hold the top 60 % of the mass
    s = Sampler(SamplerSettings(temperature=1.0, top_k=2, seed=0), "cpu")
    assert {s.sample(l) for _ in range(50)} == {1, 3}


def test_registry_and_config_reader():
    from exllamav3_amd import registry
    from exllamav3_amd.vofanex import VofanexConfig
    from exllamav3_amd.modules import GatedLinearAttention, PolyNormMLP, SlidingSinkAttention, SparseExperts
    assert {"Vofanex", "LlamaForCausalLM"} <= set(registry.architectures())
    assert registry.architecture_of({"architecture": "Vofanex"}) == "Vofanex" and registry.architecture_of({"architectures": ["LlamaForCausalLM"]}) == "LlamaForCausalLM"
    with pytest.raises(RuntimeError):
        registry.architecture_of({})
    cfg, _ = mo.random_model([dict(type="gla", heads=2, dim=8, vdim=12, tau=3.0, mlp=("moe", 8, 3, 2)),
                              dict(type="attention", heads=4, kv_heads=2, dim=8, vdim=6, window=9, scale=0.2, mlp=None),
                              dict(type="attention", heads=2, kv_heads=2, dim=4, vdim=4, window=3, mlp=("dense", 20))], width=32)
    c = VofanexConfig(json.loads(json.dumps(cfg)))
    blocks = c.build_layers()
    g, a, a2 = (b.mixer for b in blocks)
    assert isinstance(g, GatedLinearAttention) and (g.heads, g.dim, g.vdim, g.tau) == (2, 8, 12, 3.0) and abs(g.q_scale - 8 ** -0.5) < 1e-12
    assert isinstance(a, SlidingSinkAttention) and (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.scale) == (4, 2, 8, 6, 9, 0.2)
    assert isinstance(blocks[0].mlp, SparseExperts) and (blocks[0].mlp.experts, blocks[0].mlp.top, blocks[0].mlp.ff) == (3, 2, 8)
    assert blocks[1].mlp is None and isinstance(blocks[2].mlp, PolyNormMLP) and blocks[2].mlp.ff == 20
    assert c.embed_scale == cfg["embedding"]["scale"] and c.eps == cfg["norm"]["eps"]
    bad = json.loads(json.dumps(cfg)); bad["layers"][0]["type"] = "conv"
    with pytest.raises(RuntimeError):
        VofanexConfig(bad).build_layers()


def test_mixer_library_builds_and_exports_its_header():
    if not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("no hipcc")
    from exllamav3_amd import _lib
    _lib.ensure_mix_built()
    syms = _lib.check_mix_symbols()
    assert len(syms) >= 14 and _lib.mixlib().exl3_mix_abi_version() == _lib.MIX_ABI_VERSION
    l = _lib.mixlib()
    assert l.exl3_mix_topk_softmax(1, 1, 1, 4, 3, 5, None) == -1 and b"top 5 of 3" in l.exl3_mix_last_error()
    assert l.exl3_mix_gla_scan(1, 1, 1, 8, 1, 8, 1, 8, 1, 1, 1, None, 1, 1, 1, 1, 1, 300, 8, 1, 1.0, 1.0, 0, None) == -1
    with pytest.raises(RuntimeError):
        _lib.mix_check(-1)

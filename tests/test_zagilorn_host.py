"""CPU tests around the Zagilorn design: the oracle's own closed forms, the order of layer runs, the rotary frequency table of the product against the
oracle's, the registry and the declared C symbols."""
import math
import torch
import zagilorn_oracle as zo

F64 = torch.float64


def test_oracle_closed_forms():
    x = torch.tensor([[0.0, 1.0, -2.0]], dtype=F64)
    assert torch.allclose(zo.dyn_tanh(x, 0.5, torch.tensor(2.0), torch.tensor(1.0)), 2 * torch.tanh(0.5 * x) + 1)
    assert abs(float(zo.gelu_tanh(torch.tensor(1.0, dtype=F64))) - 0.8411919906082768) < 1e-12
    # a rotation keeps the length of every pair and composes: position p then q equals p + q when the magnitude is 1
    v = torch.randn(3, 2, 8, dtype=F64)
    c1, s1 = zo.rotary_tables(torch.tensor([1, 5, 9]), 6, 100.0)
    c2, s2 = zo.rotary_tables(torch.tensor([2, 2, 2]), 6, 100.0)
    c3, s3 = zo.rotary_tables(torch.tensor([3, 7, 11]), 6, 100.0)
    twice = zo.rotate_pairs(zo.rotate_pairs(v, c1, s1, 6), c2, s2, 6)
    assert torch.allclose(twice, zo.rotate_pairs(v, c3, s3, 6), atol=1e-12)
    assert torch.equal(twice[..., 6:], v[..., 6:])
    # YaRN: the fastest pairs keep their frequency, the slowest are divided by the factor, and both tables grow by 0.1 ln(factor) + 1
    sc = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}
    c, s = zo.rotary_tables(torch.tensor([1]), 16, 10000.0, sc)
    mag = 0.1 * math.log(4.0) + 1
    assert abs(float(c[0, 0] ** 2 + s[0, 0] ** 2) - mag ** 2) < 1e-12
    f = lambda i: 10000.0 ** (-2.0 * i / 16)
    assert abs(float(torch.atan2(s[0, 0], c[0, 0])) - f(0)) < 1e-12 and abs(float(torch.atan2(s[0, 7], c[0, 7])) - f(7) / 4.0) < 1e-12


def test_oracle_window_and_sink():
    T, H = 6, 1
    q = torch.zeros(T, H, 2, dtype=F64); k = torch.zeros(T, H, 2, dtype=F64)
    v = torch.arange(T, dtype=F64).reshape(T, 1, 1)
    o = zo.windowed_softmax_attention(q, k, v, 1.0, 3)
    assert torch.allclose(o[:, 0, 0], torch.tensor([0.0, 0.5, 1.0, 2.0, 3.0, 4.0], dtype=F64))          # equal scores: the mean of the last three
    o = zo.windowed_softmax_attention(q, k, v, 1.0, 3, sink=torch.zeros(1, dtype=F64))
    assert torch.allclose(o[:, 0, 0], torch.tensor([0.0, 1 / 3, 3 / 4, 6 / 4, 9 / 4, 12 / 4], dtype=F64))  # the sink is one more unit in the denominator


def test_oracle_router():
    z = torch.tensor([[2.0, 0.0, -1.0, 1.0]], dtype=F64)
    idx, w = zo.sigmoid_route(z, torch.tensor([0.0, 0.0, 5.0, 0.0], dtype=F64), 2, 3.0)
    assert sorted(idx[0].tolist()) == [0, 2]
    s = torch.sigmoid(z[0])
    assert abs(float(w.sum()) - 3.0) < 1e-12 and abs(float(w[0, idx[0].tolist().index(2)]) - 3.0 * float(s[2] / (s[0] + s[2]))) < 1e-12


def test_layer_runs_of_config_and_oracle_agree():
    from exllamav3_amd.zagilorn import ZagilornConfig
    lay = {"type": "latent_attention_2", "mixer": {}, "mlp": None}
    base = {"vocab": 8, "width": 8, "norm": {"eps": 1e-5}, "layers": [lay] * 5}
    for loop, want in ((None, [0, 1, 2, 3, 4]), ((0, 2, 3), [0, 1, 0, 1, 0, 1, 2, 3, 4]), ((1, 4, 2), [0, 1, 2, 3, 1, 2, 3, 4]), ((4, 5, 1), [0, 1, 2, 3, 4]), ((0, 5, 2), list(range(5)) * 2)):
        cfg = dict(base)
        if loop:
            cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
        runs = ZagilornConfig(cfg).runs()
        assert [i for i, _ in runs] == want and runs == zo.layer_runs(cfg)
        assert sum(1 for _, first in runs if first) == (loop[2] if loop else 0)
    for bad in ((3, 2, 1), (0, 6, 1), (0, 2, 0)):
        cfg = dict(base, loop=dict(zip(("start", "stop", "times"), bad)))
        try:
            ZagilornConfig(cfg)
            assert False, bad
        except RuntimeError:
            pass


def test_rotary_frequency_table_matches_oracle():
    from exllamav3_amd.modules import rotary_frequencies
    for dims, base, sc in ((16, 10000.0, None), (6, 300000.0, {"factor": 8.0, "original": 128, "fast": 20.0, "slow": 1.5}), (64, 1e5, {"factor": 3.0, "original": 1024, "fast": 24.0, "slow": 2.0})):
        f, mag = rotary_frequencies(dims, base, sc)
        c, s = zo.rotary_tables(torch.tensor([1]), dims, base, sc)
        assert f.dtype == torch.float32 and f.numel() == dims // 2
        assert torch.allclose(torch.atan2(s[0], c[0]), f.double(), rtol=1e-6, atol=0)                      # angle at position 1 = the frequency (all below pi here)
        assert abs(float((c[0, 0] ** 2 + s[0, 0] ** 2).sqrt()) - mag) < 1e-9


def test_registered_and_declared():
    from exllamav3_amd import _lib, registry
    assert "Zagilorn" in registry.architectures() and registry.native_libraries("Zagilorn") == ("mix",) and registry.native_libraries("Vofanex") == ("mix",)
    names = _lib.mix_declared_symbols()
    for n in ("exl3_mix_latent_prep", "exl3_mix_latent_fill_k", "exl3_mix_latent_decode", "exl3_mix_residual_norm", "exl3_mix_dyn_tanh_rows", "exl3_mix_embed_copy",
              "exl3_mix_act", "exl3_mix_glu_act", "exl3_mix_token_gate", "exl3_mix_heads_gate", "exl3_mix_topk_sigmoid", "exl3_mix_moe_gate_up_act", "exl3_mix_moe_expert_major_act"):
        assert n in names

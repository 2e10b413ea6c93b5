"""Morulix without a GPU: its configuration, the run order and tensor names that its builder makes, and what pins the
plain implementation (closed forms worked by hand)."""
import copy
import math

import pytest
import torch

import plain_morulix as pm
from morulix_util import MOR_A, MOR_B, MOR_C, MOR_D, SCALING, attention, config, latent, layer, mamba


def _spec(cfg):
    from atoma_infer_amd.config.registry import resolve_architecture
    arch = resolve_architecture(cfg)
    return arch, arch.config_cls.from_dict(copy.deepcopy(cfg))


@pytest.mark.parametrize("cfg", [MOR_A, MOR_B, MOR_C, MOR_D])
def test_configuration_reads_back_and_the_builder_names_the_checkpoint_s_tensors(cfg):
    from atoma_infer_amd.weights.loader import expected_tensors
    arch, typed = _spec(cfg)
    assert arch.name == "Morulix"
    assert arch.config_cls.from_dict(typed.to_dict()) == typed
    spec = arch.build(typed)
    names = expected_tensors(spec)
    assert {"embed", "final.norm", "head"} <= set(names)
    assert ("loop.in" in names) == ("loop" in cfg) and ("loop.step" in names) == ("loop" in cfg)
    for i, l in enumerate(cfg["layers"]):
        has = {n[len(f"l{i}."):] for n in names if n.startswith(f"l{i}.")}
        want = {"norm1"} | ({"mlp.gate", "mlp.up", "mlp.down"} if l["mlp"] else set())
        want |= {"attention": {"mix.q", "mix.k", "mix.v", "mix.o"},
                 "latent_attention": {"mix.q", "mix.dkv", "mix.dkv.norm", "mix.uk", "mix.uv", "mix.sink", "mix.g", "mix.o"},
                 "mamba2": {"mix.in", "mix.conv", "mix.conv.b", "mix.dt_bias", "mix.A_log", "mix.D", "mix.norm", "mix.o"}}[l["type"]]
        assert has == want, (i, has ^ want)
    m = cfg["layers"][0]["mixer"]
    if cfg["layers"][0]["type"] == "mamba2":
        inner = m["heads"] * m["vdim"]
        assert names["l0.mix.in"].shape == (2 * inner + 2 * m["groups"] * m["state"] + m["heads"], cfg["width"])
        assert names["l0.mix.conv"].shape == (inner + 2 * m["groups"] * m["state"], m["conv"])


def test_run_order_of_a_loop_and_a_cache_entry_for_every_pass():
    from atoma_infer_amd.cache.pool import plan_cache
    arch, typed = _spec(MOR_A)
    spec = arch.build(typed)
    entry = len(MOR_A["layers"])
    assert [c.layer for c in spec.run_order] == [0] + [entry, 1, 2] * 3
    assert [c.layer for c in spec.run_order if c.layer < entry] == [i for i, _ in pm.run_order(MOR_A)]
    plan = plan_cache(spec)
    # the window layer and the latent layer run three times each: three entries in each group; the recurrence once
    assert sorted(len(g.calls) for g in plan.groups) == [3, 3] and len(plan.states) == 1
    assert {g.spec.window for g in plan.groups} == {5, None}
    arch, typed = _spec(MOR_D)
    spec = arch.build(typed)
    assert [c.layer for c in spec.run_order] == [3, 0, 1, 3, 0, 1, 2]
    assert len(plan_cache(spec).states) == 2
    arch, typed = _spec(MOR_B)
    assert [c.layer for c in arch.build(typed).run_order] == [0, 1, 2, 3]


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][0].update(type="lstm"), "not supported"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][0]["mixer"].update(groups=2), "multiple of groups"),
    (lambda c: c["layers"][0]["mixer"].update(norm_groups=5), "norm_groups"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "not supported"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["loop"].update(times=0), "positive"),
    (lambda c: c.pop("width"), "width"),
])
def test_configurations_that_cannot_run_are_refused(change, text):
    from atoma_infer_amd.config.base import ConfigError
    cfg = copy.deepcopy(MOR_A)
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        _spec(cfg)


def test_random_weights_load_back(tmp_path):
    from atoma_infer_amd.weights import write_random_model
    from atoma_infer_amd.weights.loader import Checkpoint, check_checkpoint
    d = write_random_model(str(tmp_path / "m"), copy.deepcopy(MOR_D), seed=3, norm_jitter=0.1)
    arch, typed = _spec(MOR_D)
    ck = Checkpoint(d)
    check_checkpoint(arch.build(typed), ck)
    # norms that the design stores around zero are drawn around zero, the plain ones around one
    assert abs(float(ck.tensor("l0.norm1").float().mean())) < 0.1 and abs(float(ck.tensor("final.norm").float().mean())) < 0.1
    assert abs(float(ck.tensor("l0.mix.dkv.norm").float().mean()) - 1.0) < 0.1
    ck.close()


# ---- what pins the plain implementation ---------------------------------------------------------------------------

def test_plain_norm_and_activation():
    x = torch.tensor([[3.0, -4.0]], dtype=torch.float64)
    w = torch.tensor([0.0, 0.5], dtype=torch.float64)
    # mean square 12.5: rows over sqrt(12.5), times (1 + w)
    assert torch.allclose(pm.norm_around_zero(x, w, 0.0), torch.tensor([[3 / math.sqrt(12.5), -6 / math.sqrt(12.5)]], dtype=torch.float64))
    assert torch.allclose(pm.rms(torch.zeros(1, 4, dtype=torch.float64), 1e-6), torch.zeros(1, 4, dtype=torch.float64))
    assert abs(float(pm.silu(torch.tensor(1.0, dtype=torch.float64))) - 1 / (1 + math.exp(-1))) < 1e-15


def test_plain_frequencies_in_all_three_bands():
    f = pm.band_scaled_frequencies(10000.0, 8, None)
    assert torch.allclose(f, torch.tensor([1.0, 0.1, 0.01, 0.001], dtype=torch.float64))
    # wavelengths 6.28, 62.8, 628, 6283 against original 64, high 4, low 1: below 16 a frequency stays, above 64 it is
    # slowed by 8, between the two it is blended with s = (64 / 62.8 - 1) / (4 - 1)
    g = pm.band_scaled_frequencies(10000.0, 8, SCALING)
    s = (64 / (2 * math.pi / 0.1) - 1.0) / 3.0
    assert g[0] == f[0] and abs(float(g[2]) - 0.01 / 8) < 1e-15 and abs(float(g[3]) - 0.001 / 8) < 1e-15
    assert abs(float(g[1]) - ((1 - s) * 0.1 / 8 + s * 0.1)) < 1e-15 and 0.0125 < float(g[1]) < 0.1
    # a wavelength of 32 worked by hand: s = (64 / 32 - 1) / 3 = 1/3, so f * (2/3 / 8 + 1/3) = f * 5/12
    one = pm.band_scaled_frequencies(1.0, 2, dict(SCALING, original=64 * 2 * math.pi / 32))
    assert abs(float(one[0]) - 5.0 / 12.0) < 1e-12


def test_plain_frequency_bands_join_continuously():
    sc = {"factor": 5.0, "low": 1.0, "high": 3.0, "original": 100.0}
    def at(wavelength):
        # one frequency 2 pi / wavelength as f_0 = 1 of a table whose 'original' is rescaled to match
        return float(pm.band_scaled_frequencies(1.0, 2, dict(sc, original=100.0 * 2 * math.pi / wavelength))[0])
    lo, hi = 100.0 / 3.0, 100.0
    assert abs(at(lo * 0.9999) - 1.0) < 1e-12 and abs(at(lo * 1.0001) - 1.0) < 1e-3
    assert abs(at(hi * 1.0001) - 0.2) < 1e-12 and abs(at(hi * 0.9999) - 0.2) < 1e-3


def test_plain_rotation_pairs_signs_and_shift():
    x = torch.zeros(1, 1, 6, dtype=torch.float64)
    x[0, 0, 0] = 1.0                                    # column 0 is paired with column 2 (dims 4), columns 4, 5 pass
    x[0, 0, 5] = 7.0
    f = torch.tensor([math.pi / 2, 0.3], dtype=torch.float64)
    y = pm.rotate_halves(x, torch.tensor([1]), f)
    assert torch.allclose(y[0, 0], torch.tensor([0.0, 0.0, 1.0, 0.0, 0.0, 7.0], dtype=torch.float64), atol=1e-15)
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(3, 2, 8, generator=g, dtype=torch.float64), torch.randn(3, 2, 8, generator=g, dtype=torch.float64)
    f = pm.band_scaled_frequencies(50.0, 6, None)
    a = (pm.rotate_halves(q, torch.tensor([5, 6, 7]), f)[2] * pm.rotate_halves(k, torch.tensor([5, 6, 7]), f)[0]).sum()
    b = (pm.rotate_halves(q, torch.tensor([105, 106, 107]), f)[2] * pm.rotate_halves(k, torch.tensor([105, 106, 107]), f)[0]).sum()
    assert abs(float(a - b)) < 1e-10                    # scores depend on the distance only


def _w(spec_shapes, seed=0):
    g = torch.Generator().manual_seed(seed)
    return {k: torch.randn(*s, generator=g, dtype=torch.float64) * 0.3 for k, s in spec_shapes.items()}


def test_plain_window_of_one_key_and_two_keys_by_hand():
    m = attention(dim=4, heads=2, kv_heads=1, vdim=3, scale=0.5, window=1, rot_dims=None)
    w = _w({"a.q": (8, 5), "a.k": (4, 5), "a.v": (3, 5), "a.o": (5, 6)})
    h = torch.randn(4, 5, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    # a window of one key: softmax over the token's own key is 1, so the output is W_o [v; v]
    v = h @ w["a.v"].T
    assert torch.allclose(pm.windowed_attention(h, w, "a.", m), torch.cat([v, v], -1) @ w["a.o"].T)
    m["mask"]["size"] = 2
    out = pm.windowed_attention(h, w, "a.", m)
    q, k = (h @ w["a.q"].T).view(4, 2, 4), h @ w["a.k"].T
    s1, s2 = float(q[3, 1] @ k[2]) * 0.5, float(q[3, 1] @ k[3]) * 0.5
    p = math.exp(s1) / (math.exp(s1) + math.exp(s2))
    head1 = p * v[2] + (1 - p) * v[3]
    s1, s2 = float(q[3, 0] @ k[2]) * 0.5, float(q[3, 0] @ k[3]) * 0.5
    p = math.exp(s1) / (math.exp(s1) + math.exp(s2))
    head0 = p * v[2] + (1 - p) * v[3]
    assert torch.allclose(out[3], torch.cat([head0, head1]) @ w["a.o"].T)
    assert torch.allclose(out[0], torch.cat([v[0], v[0]]) @ w["a.o"].T)        # the first token sees itself only


def test_plain_latent_attention_first_token_and_sink_by_hand():
    m = latent(dim=4, heads=2, vdim=3, kv_rank=2, scale=0.7)
    w = _w({"a.q": (8, 5), "a.dkv": (2, 5), "a.dkv.norm": (2,), "a.uk": (8, 2), "a.uv": (6, 2), "a.sink": (2,),
            "a.g": (2, 5), "a.o": (5, 6)}, 3)
    h = torch.randn(3, 5, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    out = pm.latent_attention(h, w, "a.", m, 1e-5)
    c = h[0] @ w["a.dkv"].T
    c = c / torch.sqrt((c * c).mean() + 1e-5) * w["a.dkv.norm"]
    k, v, q = (w["a.uk"] @ c).view(2, 4), (w["a.uv"] @ c).view(2, 3), (w["a.q"] @ h[0]).view(2, 4)
    heads = []
    for hd in range(2):
        s = float(q[hd] @ k[hd]) * 0.7
        p = math.exp(s) / (math.exp(s) + math.exp(float(w["a.sink"][hd])))     # the sink: unscaled, once, no value
        heads.append(p * v[hd] / (1 + math.exp(-float(w["a.g"][hd] @ h[0]))))
    assert torch.allclose(out[0], torch.cat(heads) @ w["a.o"].T)
    w["a.sink"] = torch.full((2,), 60.0, dtype=torch.float64)                  # a sink that takes all the weight
    assert float(pm.latent_attention(h, w, "a.", m, 1e-5).abs().max()) < 1e-12


def test_plain_state_space_one_and_two_tokens_by_hand():
    m = mamba(heads=2, groups=1, vdim=2, state=3, conv=2, norm_groups=2)
    inner, gn = 4, 3
    w = _w({"a.in": (2 * inner + 2 * gn + 2, 5), "a.conv": (inner + 2 * gn, 2), "a.conv.b": (inner + 2 * gn,),
            "a.dt_bias": (2,), "a.A_log": (2,), "a.D": (2,), "a.norm": (inner,), "a.o": (5, inner)}, 4)
    h = torch.randn(2, 5, generator=torch.Generator().manual_seed(5), dtype=torch.float64)
    out = pm.mamba2(h, w, "a.", m, 1e-5)
    p = h @ w["a.in"].T
    z, raw, dtr = p[:, :inner], p[:, inner: 2 * inner + 2 * gn], p[:, 2 * inner + 2 * gn:]
    sil = lambda u: u / (1 + torch.exp(-u))
    c0 = sil(raw[0] * w["a.conv"][:, 1] + w["a.conv.b"])                       # before the start: zeros under tap 0
    c1 = sil(raw[0] * w["a.conv"][:, 0] + raw[1] * w["a.conv"][:, 1] + w["a.conv.b"])
    dt = torch.log1p(torch.exp(dtr + w["a.dt_bias"]))
    ys = []
    for hd in range(2):
        x0, x1 = c0[2 * hd: 2 * hd + 2], c1[2 * hd: 2 * hd + 2]
        b0, cc0, b1, cc1 = c0[inner: inner + 3], c0[inner + 3:], c1[inner: inner + 3], c1[inner + 3:]
        a1 = math.exp(-math.exp(float(w["a.A_log"][hd])) * float(dt[1, hd]))
        y0 = float(dt[0, hd]) * float(b0 @ cc0) * x0 + w["a.D"][hd] * x0
        y1 = a1 * float(dt[0, hd]) * float(b0 @ cc1) * x0 + float(dt[1, hd]) * float(b1 @ cc1) * x1 + w["a.D"][hd] * x1
        ys.append((y0, y1))
    for t in range(2):
        u = torch.cat([ys[0][t], ys[1][t]]) * sil(z[t])
        u = torch.cat([u[:2] / torch.sqrt((u[:2] ** 2).mean() + 1e-5), u[2:] / torch.sqrt((u[2:] ** 2).mean() + 1e-5)])
        assert torch.allclose(out[t], (u * w["a.norm"]) @ w["a.o"].T, atol=1e-12)


def test_plain_model_of_one_layer_and_the_loop_entry_by_hand():
    cfg = config([layer("attention", attention(dim=4, heads=1, kv_heads=1, scale=1.0, window=3, rot_dims=None), ff=6)],
                 width=4, vocab=5, loop=(0, 1, 2))
    w = _w({"embed": (5, 4), "loop.in": (4, 8), "loop.step": (2, 4), "l0.norm1": (4,), "l0.mix.q": (4, 4), "l0.mix.k": (4, 4),
            "l0.mix.v": (4, 4), "l0.mix.o": (4, 4), "l0.mlp.gate": (6, 4), "l0.mlp.up": (6, 4), "l0.mlp.down": (4, 6),
            "final.norm": (4,), "head": (5, 4)}, 6)
    res = []
    logits = pm.forward([3], w, cfg, res)
    e = w["embed"][3]
    x = w["loop.in"] @ torch.cat([e, e]) + w["loop.step"][0]
    def block(x):
        h = x / torch.sqrt((x * x).mean() + 1e-5) * (1 + w["l0.norm1"])
        a = w["l0.mix.o"] @ (w["l0.mix.v"] @ h)                                 # one token: the softmax is 1
        g = w["l0.mlp.gate"] @ h
        return x + a + w["l0.mlp.down"] @ (g / (1 + torch.exp(-g)) * (w["l0.mlp.up"] @ h))
    x1 = block(x)
    x2 = block(w["loop.in"] @ torch.cat([x1, e]) + w["loop.step"][1])          # the second pass reads the embedding again
    assert len(res) == 2 and torch.allclose(res[0][0], x1) and torch.allclose(res[1][0], x2)
    assert torch.allclose(logits[0], w["head"] @ (x2 / torch.sqrt((x2 * x2).mean() + 1e-5) * (1 + w["final.norm"])))


def test_plain_model_does_not_look_ahead():
    from atoma_infer_amd.weights import write_random_model
    import os, tempfile
    from safetensors.torch import load_file
    with tempfile.TemporaryDirectory() as d:
        write_random_model(d, copy.deepcopy(MOR_A), seed=1, norm_jitter=0.1)
        w = {k: v.double() for k, v in load_file(os.path.join(d, "model.safetensors")).items()}
    a = pm.forward([1, 2, 3, 4, 5, 6, 7, 8], w, MOR_A)
    b = pm.forward([1, 2, 3, 4, 5, 9, 9, 9], w, MOR_A)
    assert torch.allclose(a[:5], b[:5]) and not torch.allclose(a[5], b[5])

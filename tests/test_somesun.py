"""Somesun on the CPU: its configuration and tensor names, and what pins the plain implementation beside its text."""
import math

import pytest
import torch

import plain_somesun as ps
from atoma_infer_amd.cache.pool import plan_cache
from atoma_infer_amd.config import ConfigError
from atoma_infer_amd.config.registry import resolve_architecture
from atoma_infer_amd.kernels import attention_bf16
from atoma_infer_amd.weights.loader import expected_tensors
from somesun_util import SUN_A, SUN_B, layer


def build(cfg):
    arch = resolve_architecture(cfg)
    typed = arch.config_cls.from_dict(cfg)
    return arch, typed, arch.build(typed)


def test_the_architecture_key_selects_the_design_and_the_configuration_round_trips():
    arch, typed, spec = build(SUN_A)
    assert arch.name == "Somesun" and len(typed.layers) == 2
    assert arch.config_cls.from_dict(typed.to_dict()) == typed
    l0, l1 = typed.layers
    assert (l0.mixer.left.mask.size, l0.mixer.left.rot.dims, l0.mlp.top) == (7, 16, 2)
    assert l1.mlp is None and l1.mixer.right.conv == 4


def test_tensor_names_and_shapes_follow_every_layer_s_own_sizes():
    _, _, spec = build(SUN_A)
    want = expected_tensors(spec)
    assert want["embed"].shape == (97, 64) and want["head"].shape == (97, 64) and want["final.norm"].shape == (64,)
    assert want["l0.mix.left.q"].shape == (4 * 32, 64) and want["l0.mix.left.k"].shape == (2 * 32, 64)
    assert want["l0.mix.left.q.norm"].shape == (128,) and want["l0.mix.left.sink"].shape == (4,)
    assert "l0.mix.left.v" not in want                       # the values are the keys
    assert want["l0.mix.right.q"].shape == (2 * 16, 64) and want["l0.mix.right.v"].shape == (4 * 24, 64)
    assert want["l0.mix.right.q.conv"].shape == (32, 3) and want["l0.mix.right.dt_bias"].shape == (4 * 16,)
    assert want["l0.mix.right.a1"].shape == (5, 64) and want["l0.mix.right.a2"].shape == (64, 5)      # named in SUN_A
    assert want["l1.mix.right.a1"].shape == (-1, 64) and want["l1.mix.right.a1"].fits((9, 64))       # the checkpoint's
    assert want["l0.mlp.router"].shape == (4, 64) and want["l0.mlp.e3.down"].shape == (64, 48)
    assert "l1.mlp.router" not in want and "l1.norm2" not in want and "l1.norm1b" in want
    plan = plan_cache(spec)
    # a cache group per key geometry, a state per layer: convolution inputs and S
    assert len(plan.groups) == 2
    assert plan.states[0] == (((3 - 1) * (2 * 32 + 96) + 4 * 24 * 16,), "float32")


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][0]["mixer"]["left"].update(vdim=16), "values are the keys"),
    (lambda c: c["layers"][0].update(type="serial"), "not supported"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "exceeds"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=34), "rotated columns"),
    (lambda c: c["norm"].update(eps=0.0), "positive"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(kv_heads=3), "multiple"),
])
def test_configurations_that_cannot_run_are_refused(change, text):
    import copy
    cfg = copy.deepcopy(SUN_A)
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        build(cfg)


def test_the_planner_s_first_key_under_windows_and_chunks():
    import numpy as np
    pos = np.arange(0, 40)
    assert (attention_bf16.first_key(pos, 0) == 0).all()
    assert (attention_bf16.first_key(pos, 5) == np.maximum(0, pos - 4)).all()
    assert (attention_bf16.first_key(pos, -7) == (pos // 7) * 7).all()
    # a decoded token's tasks start at its chunk's first key (rounded down to a block of 32 keys), wherever it stands
    arr, meta = attention_bf16.build_tasks(np.asarray([99, 100, 7]), np.asarray([1, 1, 1]), 2, -50, 256, kv_heads=1,
                                           max_waves=8, head_size=64)
    main = arr[: meta[0]]
    live = main[main[:, 0] >= 0]
    assert sorted(zip(live[:, 0].tolist(), live[:, 4].tolist(), live[:, 5].tolist())) == [(0, 32, 100), (1, 96, 101), (2, 0, 8)]


# ---- what pins the plain implementation -------------------------------------------------------------------------

def test_plain_rotation_is_a_turn_of_neighbouring_pairs():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 3, 8, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 10, 1000])
    y = ps.rotate_pairs(x, pos, 100.0, 4)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 4:], x[..., 4:])          # position 0; columns beyond dims
    a = 10 * 100.0 ** (-2 * 1 / 4)                                                   # pair 1 of position 10
    u, v = x[3, 2, 2], x[3, 2, 3]
    assert torch.allclose(y[3, 2, 2], u * math.cos(a) - v * math.sin(a)) and \
        torch.allclose(y[3, 2, 3], v * math.cos(a) + u * math.sin(a))
    # scores depend on the distance only
    q, k = torch.randn(1, 1, 8, generator=g, dtype=torch.float64), torch.randn(1, 1, 8, generator=g, dtype=torch.float64)
    d1 = (ps.rotate_pairs(q, torch.tensor([7]), 50.0, 8) * ps.rotate_pairs(k, torch.tensor([3]), 50.0, 8)).sum()
    d2 = (ps.rotate_pairs(q, torch.tensor([107]), 50.0, 8) * ps.rotate_pairs(k, torch.tensor([103]), 50.0, 8)).sum()
    assert torch.allclose(d1, d2)


def _one_layer(width=8):
    return {"left": {"dim": 4, "heads": 2, "kv_heads": 1, "vdim": 4, "scale": 0.5, "mask": {"size": 3},
                     "rot": {"base": 10.0, "dims": 2}},
            "right": {"dim": 4, "heads": 2, "kv_heads": 1, "vdim": 3, "conv": 2}}


def test_plain_attention_of_one_token_is_its_value_shared_with_the_sink():
    m = _one_layer()["left"]
    g = torch.Generator().manual_seed(1)
    w = {"a.q": torch.randn(8, 8, generator=g, dtype=torch.float64), "a.k": torch.randn(4, 8, generator=g, dtype=torch.float64),
         "a.q.norm": torch.rand(8, generator=g, dtype=torch.float64) + 0.5,
         "a.k.norm": torch.rand(4, generator=g, dtype=torch.float64) + 0.5,
         "a.sink": torch.tensor([0.3, -1.2], dtype=torch.float64), "a.o": torch.eye(8, dtype=torch.float64)}
    h = torch.randn(1, 8, generator=g, dtype=torch.float64)
    out = ps.chunked_sink_attention(h, w, "a.", m, 1e-5)
    q, k = w["a.q"] @ h[0], w["a.k"] @ h[0]
    qn = q / torch.sqrt((q * q).mean() + 1e-5) * w["a.q.norm"]
    kn = k / torch.sqrt((k * k).mean() + 1e-5) * w["a.k.norm"]
    for head in range(2):
        s = (qn[4 * head: 4 * head + 4] * kn).sum() * 0.5                 # position 0: no turn
        share = torch.exp(s) / (torch.exp(s) + torch.exp(w["a.sink"][head]))
        assert torch.allclose(out[0, 4 * head: 4 * head + 4], share * k)  # the value is k as projected


def test_plain_attention_forgets_at_a_chunk_s_first_position():
    m = _one_layer()["left"]
    g = torch.Generator().manual_seed(2)
    w = {"a.q": torch.randn(8, 8, generator=g, dtype=torch.float64), "a.k": torch.randn(4, 8, generator=g, dtype=torch.float64),
         "a.q.norm": torch.ones(8, dtype=torch.float64), "a.k.norm": torch.ones(4, dtype=torch.float64),
         "a.sink": torch.zeros(2, dtype=torch.float64), "a.o": torch.eye(8, dtype=torch.float64)}
    h = torch.randn(7, 8, generator=g, dtype=torch.float64)
    out = ps.chunked_sink_attention(h, w, "a.", m, 1e-5)
    h2 = h.clone()
    h2[:3] = torch.randn(3, 8, generator=g, dtype=torch.float64)          # the first chunk (size 3) changed
    out2 = ps.chunked_sink_attention(h2, w, "a.", m, 1e-5)
    assert torch.allclose(out[3:], out2[3:]) and not torch.allclose(out[2], out2[2])
    h3 = h.clone()
    h3[3] += 1.0                                                          # position 3 is seen by 3, 4, 5 and not by 6
    out3 = ps.chunked_sink_attention(h3, w, "a.", m, 1e-5)
    assert torch.allclose(out[6], out3[6]) and not torch.allclose(out[5], out3[5])


def test_plain_convolution_and_delta_rule_in_closed_form():
    x = torch.tensor([[1.0, -2.0], [0.5, 3.0], [2.0, 1.0]], dtype=torch.float64)
    taps = torch.tensor([[0.5, 2.0], [1.0, -1.0]], dtype=torch.float64)                # last column: the current token
    y = ps.causal_conv_silu(x, taps)
    pre = torch.tensor([[2.0, 2.0], [0.5 * 1 + 2 * 0.5, -2.0 - 3.0], [0.5 * 0.5 + 4.0, 3.0 - 1.0]], dtype=torch.float64)
    assert torch.allclose(y, pre * torch.sigmoid(pre))
    # one token through the recurrence: S = k u^T with u = beta v, read with q: o = (k . q) beta v
    m = _one_layer()["right"]
    g = torch.Generator().manual_seed(3)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = {"r.q": r(4, 8), "r.k": r(4, 8), "r.v": r(6, 8), "r.q.conv": r(4, 2), "r.k.conv": r(4, 2), "r.v.conv": r(6, 2),
         "r.b": r(2, 8), "r.a1": r(3, 8), "r.a2": r(8, 3), "r.dt_bias": r(8), "r.A_log": r(2), "r.g1": r(3, 8),
         "r.g2": r(6, 3), "r.norm": torch.rand(3, generator=g, dtype=torch.float64) + 0.5, "r.o": torch.eye(8, 6, dtype=torch.float64)}
    h = r(1, 8)
    out = ps.gated_delta(h, w, "r.", m, 1e-5)
    act = lambda name: ps.silu((w["r." + name] @ h[0]) * w[f"r.{name}.conv"][:, -1])
    q, k, v = act("q"), act("k"), act("v").view(2, 3)
    q = q / torch.sqrt((q * q).sum() + 1e-6) / 2.0
    k = k / torch.sqrt((k * k).sum() + 1e-6)
    beta = torch.sigmoid(w["r.b"] @ h[0])
    gate = torch.sigmoid(w["r.g2"] @ (w["r.g1"] @ h[0])).view(2, 3)
    for head in range(2):
        o = (k @ q) * beta[head] * v[head]
        o = o / torch.sqrt((o * o).mean() + 1e-5) * w["r.norm"] * gate[head]
        assert torch.allclose(out[0, 3 * head: 3 * head + 3], o)


def test_plain_delta_rule_decays_per_key_channel_and_writes_before_it_reads():
    # two tokens by hand, one head, dim 2, vdim 1, no convolution history (taps 1): S1 = k1 u1^T; then
    # S2 = g2 * S1 + k2 u2^T with u2 = beta2 (v2 - (g2 * S1)^T k2), read with q2
    g1, g2 = torch.tensor([0.5, 0.25], dtype=torch.float64), torch.tensor([0.8, 0.1], dtype=torch.float64)
    k1, k2 = torch.tensor([1.0, 0.0], dtype=torch.float64), torch.tensor([0.6, 0.8], dtype=torch.float64)
    q2 = torch.tensor([0.3, -0.4], dtype=torch.float64)
    v1, v2, b1, b2 = 2.0, -1.0, 0.5, 0.9
    s = torch.zeros(2, 1, dtype=torch.float64)
    s = g1[:, None] * s
    s = s + torch.outer(k1, torch.tensor([b1 * (v1 - float(s[:, 0] @ k1))], dtype=torch.float64))
    s = g2[:, None] * s
    u2 = b2 * (v2 - float(s[:, 0] @ k2))
    s = s + torch.outer(k2, torch.tensor([u2], dtype=torch.float64))
    by_hand = float(s[:, 0] @ q2)
    assert abs(by_hand - (0.8 * 1.0 * 0.3 + u2 * (0.6 * 0.3 - 0.8 * 0.4))) < 1e-12     # S1 = [[1], [0]]


def test_plain_experts_weigh_the_input_not_the_output():
    g = torch.Generator().manual_seed(4)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = {"m.router": torch.tensor([[0.0] * 4, [1.0] * 4, [-1.0] * 4], dtype=torch.float64)}
    for e in range(3):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"], w[f"m.e{e}.down"] = r(5, 4), r(5, 4), r(4, 5)
    h = torch.tensor([[0.5, 0.5, 0.5, 0.5]], dtype=torch.float64)              # logits 0, 2, -2: experts 1 and 0
    out = ps.routed_experts(h, w, "m.", {"router": {"experts": 3, "top": 2}})
    want = 0
    for e, z in ((1, 2.0), (0, 0.0)):
        x = torch.sigmoid(torch.tensor(z, dtype=torch.float64)) * h[0]
        want = want + w[f"m.e{e}.down"] @ (ps.silu(w[f"m.e{e}.gate"] @ x) * (w[f"m.e{e}.up"] @ x))
    assert torch.allclose(out[0], want)
    assert not torch.allclose(out[0], sum(torch.sigmoid(torch.tensor(z, dtype=torch.float64)) *
                                          (w[f"m.e{e}.down"] @ (ps.silu(w[f"m.e{e}.gate"] @ h[0]) * (w[f"m.e{e}.up"] @ h[0])))
                                          for e, z in ((1, 2.0), (0, 0.0))))


def test_plain_layer_without_a_feed_forward_and_layer_helper():
    assert layer(left=dict(dim=8))["mixer"]["left"]["dim"] == 8 and layer(mlp=None)["mlp"] is None


def test_pages_behind_a_token_s_chunk_go_back_while_the_request_runs():
    from atoma_infer_amd.cache.manager import CacheManager, GroupGeometry
    m = CacheManager([GroupGeometry(16, 12, None, 40)], 2)
    m.add(7)
    m.reserve(7, 100)
    assert m.table(7) == [0, 1, 2, 3, 4, 5, 6]
    # the token at position 100 sees keys 80 .. 100: the five pages wholly below 80 are dead
    assert m.release_behind(7, 100) == 5 and m.table(7) == [-1] * 5 + [5, 6]
    assert m.release_behind(7, 119) == 0             # still in the chunk that began at 80
    m.reserve(7, 121)
    # position 120 opens a chunk in the middle of a page, which stays; the pages before it go
    assert m.release_behind(7, 120) == 2 and m.table(7)[:7] == [-1] * 7 and m.table(7)[7] >= 0
    m.check()
    m.free(7)
    m.check()
    assert m.num_free_pages() == 12
    _, _, spec = build(SUN_A)
    assert [g.spec.chunk for g in plan_cache(spec).groups] == [7, 16]

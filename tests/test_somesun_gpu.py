"""Somesun on the GPU against the plain implementation: every mechanism, then the whole model through the runner's
step function (portions, batches, pages and slots used again) and through the engine's own entry point."""
import types

import numpy as np
import pytest
import torch

import plain_somesun as ps
from somesun_util import (SUN_A, SUN_B, SUN_C, TOL, assert_logits, config, layer, logit_err, make_runner, plain_config, plain_weights,
                          run_schedule, tokens, write_model)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("somesun")
    return {"A": write_model(str(root / "a"), SUN_A, 11), "B": write_model(str(root / "b"), SUN_B, 12),
            "C": write_model(str(root / "c"), SUN_C, 13)}


def oracle(path, toks):
    return ps.forward(list(toks), plain_weights(path), plain_config(path)).float()


# ---- mechanisms alone -----------------------------------------------------------------------------------------

@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, planes", [(64, (1, 1)), (200, (2, 3)), (4100, (1, 0))])
def test_sum_and_norm_behind_a_sublayer(width, planes, out_dtype):
    from atoma_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(width)
    t = 5
    resid = torch.randn(t, width, generator=g)
    a = torch.randn(planes[0], t, width, generator=g)
    terms = [(a, 0.6)]
    if planes[1]:
        terms.append((torch.randn(planes[1], t, width, generator=g).to(torch.bfloat16), -1.7))
    wp, wn = torch.rand(width, generator=g) + 0.5, torch.rand(width, generator=g) + 0.5
    d = sum(x.double().sum(0) * s for x, s in terms)
    want_resid = resid.double() + ps.rms_norm(d, wp.double(), 1e-5)
    want_out = ps.rms_norm(want_resid, wn.double(), 2e-6)
    r = resid.to(DEV)
    dev_terms = [((x[0] if x.shape[0] == 1 else x).contiguous().to(DEV), s) for x, s in terms]
    out = ops.add_normed(r, dev_terms, wp.to(DEV), 1e-5, wn.to(DEV), 2e-6, out_dtype)
    assert (r.cpu().double() - want_resid).abs().max() < 2e-5
    assert (out.cpu().double() - want_out).abs().max() < (2e-5 if out_dtype is torch.float32 else 3e-2)
    r2 = resid.to(DEV)
    assert ops.add_normed(r2, dev_terms, wp.to(DEV), 1e-5) is None and torch.equal(r2, r)


def _ctx(starts, counts, slots):
    """What a mixer reads of a step, for entries of ``counts`` tokens at ``starts``, built by hand."""
    t = int(sum(counts))
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    seq = [e for e, c in enumerate(counts) for _ in range(c)]
    pos = [s + j for s, c in zip(starts, counts) for j in range(c)]
    q_start = np.concatenate([[0], np.cumsum(counts)]).tolist()
    return types.SimpleNamespace(n_tokens=t, n_entries=len(counts), positions=i32(pos), token_seq=i32(seq),
                                 q_start=i32(q_start), state_slots=i32(slots), h_starts=np.asarray(starts, dtype=np.int32),
                                 h_counts=np.asarray(counts, dtype=np.int32), plans={}, scratch={}, decode_bucket=None)


def _load(part, weights, dtype):
    part.load(lambda name: weights[name].to(torch.bfloat16), torch.device(DEV), dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, taps", [(4, 2, 16, 24, 3), (2, 2, 40, 8, 4), (3, 1, 128, 40, 1),
                                                              (1, 1, 200, 5, 2)])
def test_gated_delta_rule_alone_whole_and_in_portions(heads, kv_heads, dim, vdim, taps, dtype):
    """The mixer on hand-made steps: two requests side by side, cut into portions of unequal lengths (one token, two,
    fewer than the convolution has taps, many), each carried by its state slot; against the plain recurrence."""
    from atoma_infer_amd.parts import GatedDeltaRule
    from atoma_infer_amd.weights.random_init import random_tensor
    width = 64
    part = GatedDeltaRule(width, heads, kv_heads, dim, vdim, taps, 1e-5, decay_rank=6, gate_rank=7)
    w = {n: random_tensor("x." + n, ws, 5, torch.bfloat16).float() for n, ws in part.weight_specs().items()}
    w["o"] = (w["o"] * 20).to(torch.bfloat16).float()                      # outputs of order one
    _load(part, w, dtype)
    g = torch.Generator().manual_seed(dim)
    lens = (37, 9)
    hs = [torch.randn(n, width, generator=g).to(torch.bfloat16).float() for n in lens]
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps}
    want = [ps.gated_delta(h.double(), {"r." + k: v.double() for k, v in w.items()}, "r.", m, 1e-5) for h in hs]
    state = torch.zeros((4, part.state_spec().shape[0]), dtype=torch.float32, device=DEV)
    state[1].fill_(7.0)                       # another request's slot must stay as it is
    cache = types.SimpleNamespace(state=state)
    got = [[], []]
    at = [0, 0]
    for cuts in ([(0, 1), (1, 2)], [(0, 2)], [(1, 1), (0, 1)], [(0, 30), (1, 6)], [(0, 3)]):
        ctx = _ctx([at[r] for r, _ in cuts], [n for _, n in cuts], [3 if r == 0 else 0 for r, _ in cuts])
        x = torch.cat([hs[r][at[r]: at[r] + n] for r, n in cuts]).to(DEV, dtype)
        y = part.forward(x, ctx, cache)
        y = (y.sum(0) if y.dim() == 3 else y).float().cpu()
        o = 0
        for r, n in cuts:
            got[r].append(y[o: o + n])
            o += n
            at[r] += n
    assert at == list(lens) and bool((state[1] == 7.0).all())
    tol = 2e-5 if dtype is torch.float32 else 3e-2
    for r in range(2):
        err = (torch.cat(got[r]).double() - want[r]).norm() / want[r].norm()
        assert err < tol, (r, float(err))


def test_a_far_token_stays_in_the_recurrent_state():
    """Decays close to one and one early token whose value is large: hundreds of tokens later the read-out still
    holds it.  A state that is lost, cleared or carried by the wrong slot changes the late outputs entirely."""
    from atoma_infer_amd.parts import GatedDeltaRule
    from atoma_infer_amd.weights.random_init import random_tensor
    width, heads, dim, vdim, taps = 64, 2, 32, 16, 2
    part = GatedDeltaRule(width, heads, 2, dim, vdim, taps, 1e-5, decay_rank=4, gate_rank=4)
    w = {n: random_tensor("y." + n, ws, 9, torch.bfloat16).float() for n, ws in part.weight_specs().items()}
    w["dt_bias"] = torch.full_like(w["dt_bias"], -9.0)           # softplus(-9) = 1.2e-4: the state hardly decays
    w["a2"] = w["a2"] * 0
    w["o"] = (w["o"] * 20).to(torch.bfloat16).float()
    _load(part, w, torch.float32)
    g = torch.Generator().manual_seed(1)
    n = 400
    h = torch.randn(n, width, generator=g).to(torch.bfloat16).float() * 0.3
    h[5] = h[5] * 40                                              # the far token
    m = {"heads": heads, "kv_heads": 2, "dim": dim, "vdim": vdim, "conv": taps}
    pw = {"r." + k: v.double() for k, v in w.items()}
    want = ps.gated_delta(h.double(), pw, "r.", m, 1e-5)
    h_without = h.clone()
    h_without[5] = h[5] / 40
    assert (ps.gated_delta(h_without.double(), pw, "r.", m, 1e-5)[-20:] - want[-20:]).norm() > 0.2 * want[-20:].norm()
    state = torch.zeros((2, part.state_spec().shape[0]), dtype=torch.float32, device=DEV)
    cache = types.SimpleNamespace(state=state)
    got, at = [], 0
    for c in [300, 63, 2] + [1] * 35:
        y = part.forward(h[at: at + c].to(DEV), _ctx([at], [c], [1]), cache)
        got.append((y.sum(0) if y.dim() == 3 else y).float().cpu())
        at += c
    got = torch.cat(got)
    assert (got.double() - want).norm() / want.norm() < 2e-5
    assert (got[-20:].double() - want[-20:]).norm() / want[-20:].norm() < 2e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts, top, ff", [(4, 2, 48), (3, 1, 64), (5, 5, 24), (70, 3, 16), (6, 2, 96), (40, 4, 32)])
def test_routed_experts_alone(experts, top, ff, dtype):
    from atoma_infer_amd.parts import RoutedExperts
    from atoma_infer_amd.weights.random_init import random_tensor
    width = 96
    part = RoutedExperts(width, ff, experts, top)
    w = {n: random_tensor("z." + n, ws, 3, torch.bfloat16).float() for n, ws in part.weight_specs().items()}
    for n in w:
        if n != "router":
            w[n] = (w[n] * 10).to(torch.bfloat16).float()
    _load(part, w, dtype)
    # (the matrix-core products take expert widths that are multiples of 32 in bfloat16; the others, and the 32-bit
    # path, run float32 multiply-adds)
    assert part.mfma == (dtype is torch.bfloat16 and ff % 32 == 0)
    g = torch.Generator().manual_seed(experts)
    for t in (1, 3, 150, 700):     # one row tile, experts whose rows fill more than one, tiles of 128 places
        h = torch.randn(t, width, generator=g).to(torch.bfloat16).float()
        want = ps.routed_experts(h.double(), {"m." + k: v.double() for k, v in w.items()}, "m.",
                                 {"router": {"experts": experts, "top": top}})
        got = part.forward(h.to(DEV, dtype), None)
        assert tuple(got.shape) == (top, t, width)
        err = (got.sum(0).cpu().double() - want).norm() / want.norm()
        assert err < (2e-5 if dtype is torch.float32 else 2e-2), (t, float(err))


def _attention_case(dtype, hd, nh, nkv, chunk, rot, lens_and_cuts, page, sink_value=None, boost=None, scale=0.3):
    """The attention mixer alone on hand-made steps over a paged cache whose pages are dealt out of order."""
    from atoma_infer_amd.parts import TiedValueAttention
    from atoma_infer_amd.weights.random_init import random_tensor
    width = 64
    part = TiedValueAttention(width, nh, nkv, hd, scale, 1e-5, 300.0, rot, chunk=chunk)
    w = {n: random_tensor("t." + n, ws, 7, torch.bfloat16).float() for n, ws in part.weight_specs().items()}
    w["q"], w["k"] = (w["q"] * 30).to(torch.bfloat16).float(), (w["k"] * 30).to(torch.bfloat16).float()
    w["o"] = (torch.eye(width, nh * hd) + w["o"]).to(torch.bfloat16).float()
    if sink_value is not None:
        w["sink"] = torch.full_like(w["sink"], sink_value)
    _load(part, w, dtype)
    lens = [sum(c for r2, c in sum(lens_and_cuts, []) if r2 == r) for r in range(2)]
    g = torch.Generator().manual_seed(hd + chunk)
    hs = [torch.randn(n, width, generator=g).to(torch.bfloat16).float() for n in lens]
    if boost is not None:
        # one position whose key every later query of the request scores far above all others, if it may see it
        r, p = boost
        hs[r][p + 1:] = (hs[r][p + 1:] * 0.2 + hs[r][p] * 3).to(torch.bfloat16).float()
    m = {"heads": nh, "kv_heads": nkv, "dim": hd, "vdim": hd, "scale": scale, "mask": {"size": chunk},
         "rot": {"base": 300.0, "dims": rot}}
    want = [ps.chunked_sink_attention(h.double(), {"a." + k: v.double() for k, v in w.items()}, "a.", m, 1e-5)
            for h in hs if len(h)]
    n_pages = sum(-(-n // page) for n in lens) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    tables = [[order.pop() for _ in range(-(-n // page))] for n in lens]
    max_blocks = max(len(tb) for tb in tables)
    cdt = dtype
    k = torch.zeros((n_pages, nkv, page * part.hd), dtype=cdt, device=DEV)      # (part.hd: the size the kernels see)
    v = torch.zeros_like(k)
    got, at = [[], []], [0, 0]
    for cuts in lens_and_cuts:
        ctx = _ctx([at[r] for r, _ in cuts], [n for _, n in cuts], [0] * len(cuts))
        bt = torch.tensor([tables[r] + [0] * (max_blocks - len(tables[r])) for r, _ in cuts], dtype=torch.int32, device=DEV)
        slots = [tables[r][(at[r] + j) // page] * page + (at[r] + j) % page for r, n in cuts for j in range(n)]
        cache = types.SimpleNamespace(k=k, v=v, page_size=page, writable=True, block_tables=bt,
                                      slot_mapping=torch.tensor(slots, dtype=torch.int32, device=DEV))
        x = torch.cat([hs[r][at[r]: at[r] + n] for r, n in cuts]).to(DEV, dtype)
        y = part.forward(x, ctx, cache)
        y = (y.sum(0) if y.dim() == 3 else y).float().cpu()
        o = 0
        for r, n in cuts:
            got[r].append(y[o: o + n])
            o += n
            at[r] += n
    return [torch.cat(x) for x in got if x], want


CUTS = [[(0, 20), (1, 3)], [(0, 1), (1, 1)], [(0, 2)], [(1, 40), (0, 1)], [(0, 50)], [(0, 1)], [(1, 1)], [(0, 1), (1, 2)]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hd, nh, nkv, chunk, rot, page", [(32, 4, 2, 7, 16, 16), (64, 8, 2, 33, 64, 16), (48, 2, 1, 16, 48, 32),
                                                           (64, 4, 4, 1, 0, 16), (24, 3, 1, 1000, 24, 4),
                                                           (20, 3, 1, 9, 10, 16), (36, 2, 2, 50, 36, 32)])
def test_tied_value_attention_alone(hd, nh, nkv, chunk, rot, page, dtype):
    """Head sizes that are multiples of 16 and others (run as the next multiple of 16, zeros in the added columns); chunks of one position and chunks longer
    than the requests; no column rotated, some, all; pages of 4, 16 and 32 tokens."""
    got, want = _attention_case(dtype, hd, nh, nkv, chunk, rot, CUTS, page)
    for a, b in zip(got, want):
        err = (a.double() - b).norm() / b.norm()
        assert err < (2e-5 if dtype is torch.float32 else 2.5e-2), float(err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("edge", [-1, 0])
def test_a_dominant_key_just_outside_and_just_inside_a_chunk(dtype, edge):
    """A key that outweighs all others stands at a chunk's last position (just outside for the next chunk's tokens) or at
    a chunk's first (just inside): a mask that is one position off changes every later row of that chunk."""
    chunk = 24
    p = 2 * chunk + edge
    got, want = _attention_case(dtype, 64, 4, 1, chunk, 64, [[(0, 30), (1, 5)], [(0, 30)], [(0, 1)], [(0, 2)]] +
                                [[(0, 1)]] * 20, 16, boost=(0, p), scale=0.6)
    rows = slice(p + 1, 3 * chunk - 1)
    err = (got[0][rows].double() - want[0][rows]).norm() / want[0][rows].norm()
    assert err < (2e-5 if dtype is torch.float32 else 3e-2), float(err)
    assert (got[0].double() - want[0]).norm() / want[0].norm() < (2e-5 if dtype is torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sink", [-30.0, 0.0, 6.0])
def test_the_sink_takes_its_share(sink, dtype):
    """A sink far below the scores changes nothing, one far above takes nearly all of the weight."""
    got, want = _attention_case(dtype, 64, 4, 2, 40, 32, CUTS, 16, sink_value=sink)
    for a, b in zip(got, want):
        assert (a.double() - b).norm() / b.norm() < (2e-5 if dtype is torch.float32 else 2.5e-2)
    if sink != 0.0:
        zero, _ = _attention_case(dtype, 64, 4, 2, 40, 32, CUTS, 16, sink_value=0.0)
        assert (got[0] - zero[0]).norm() > 0.05 * zero[0].norm()


@pytest.mark.parametrize("second_kernel", [False, True])
def test_sinks_and_chunks_where_a_token_s_keys_are_cut_into_parts(monkeypatch, second_kernel):
    """Long chunks in bfloat16: decoded tokens and short portions late in a chunk have their keys cut into parts that
    are merged by the attention kernel or by the merging kernel; the sink joins the denominator once, at the merge."""
    from util import force_chunked_decode
    force_chunked_decode(monkeypatch, second_kernel)
    cuts = [[(0, 700), (1, 300)], [(0, 3), (1, 1)], [(0, 1), (1, 1)], [(0, 1)], [(0, 330), (1, 1)], [(0, 1), (1, 1)],
            [(0, 2)], [(0, 1)]]
    got, want = _attention_case(torch.bfloat16, 64, 8, 2, 1024, 64, cuts, 16, sink_value=2.0)
    for a, b in zip(got, want):
        assert (a.double() - b).norm() / b.norm() < 2.5e-2
        assert (a[-6:].double() - b[-6:]).norm() / b[-6:].norm() < 2.5e-2


# ---- the whole model through the step function --------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_prompts_token_by_token_decoding_and_portions(dirs, name, dtype):
    d = dirs[name]
    vocab = plain_config(d)["vocab"]
    toks = tokens(150, vocab, 3)
    want = oracle(d, toks)
    runner = make_runner(d, dtype, 256, 16, 4)
    n = len(toks)
    schedules = {
        "whole": [[(0, n)]],
        "tokens": [[(0, 1)]] * n,                                        # crosses every chunk edge one token at a time
        "portions": [[(0, c)] for c in (2, 2, 3, 1, 16, 2, 31, 33, 2, 7, 1, 1, 2, 40, 7)],
        "long decoding": [[(0, 10)]] + [[(0, 1)]] * (n - 10),
    }
    assert sum(c for s in schedules["portions"] for _, c in s) == n
    for what, sched in schedules.items():
        got = run_schedule(runner, {0: toks}, sched)[0]
        assert_logits(got, want, dtype, what)
    runner.manager.check()
    assert runner.manager.num_requests() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_batches_of_unequal_requests_with_pages_and_slots_used_again(dirs, name, dtype):
    """Up to four live requests, portions beside single tokens, in a pool that holds them only because finished requests
    give their pages and state slots back: every request's logits are those of the request alone."""
    d = dirs[name]
    vocab = plain_config(d)["vocab"]
    reqs = {i: tokens(n, vocab, 20 + i) for i, n in enumerate((70, 1, 45, 130, 2, 64, 33))}
    want = {i: oracle(d, t) for i, t in reqs.items()}
    sched = [[(0, 30), (1, 1)], [(0, 1), (2, 2), (3, 64)], [(0, 1), (2, 1), (3, 2), (4, 1)], [(0, 38), (2, 42), (4, 1)],
             [(3, 1), (5, 17)], [(3, 33), (5, 1), (6, 2)], [(5, 46), (6, 1), (3, 1)], [(6, 30), (3, 29)]]
    runner = make_runner(d, dtype, 320, 16, 4)      # 345 tokens in all: only with pages used again
    got = run_schedule(runner, reqs, sched)
    for i in reqs:
        assert_logits(got[i], want[i], dtype, i)
    runner.manager.check()
    assert runner.manager.num_requests() == 0 and runner.manager.num_free_slots() == 4


def test_decode_steps_replayed_as_graphs_give_the_eager_logits(dirs):
    """Steps in which every entry brings one token are recorded into graphs from their second sighting on; the
    recurrent state, the convolution's inputs and the experts' grouping are read from the step's device tensors."""
    d = dirs["B"]
    vocab = plain_config(d)["vocab"]
    reqs = {i: tokens(60, vocab, 40 + i) for i in range(3)}
    want = {i: oracle(d, t) for i, t in reqs.items()}
    sched = [[(0, 20), (1, 5), (2, 9)]] + [[(0, 1), (1, 1), (2, 1)]] * 40 + [[(1, 15)], [(2, 11)]]
    runner = make_runner(d, "bfloat16", 256, 16, 4)
    assert runner.use_graphs
    got = run_schedule(runner, reqs, sched)
    assert any(g.graph is not None for g in runner._graphs.values())
    for i in reqs:
        assert_logits(got[i], want[i], "bfloat16", i)


def test_a_lone_prompt_s_step_replayed_as_a_graph(dirs):
    """A step that is one prompt of 256 tokens or more and wants its last place is recorded the third time its shape is
    seen: every replay, with other tokens and another state slot, gives what a runner without graphs gives."""
    from atoma_infer_amd.engine.step import StepEntry
    d = dirs["B"]
    vocab = plain_config(d)["vocab"]
    runner = make_runner(d, "bfloat16", 1024, 16, 4)
    eager = make_runner(d, "bfloat16", 1024, 16, 4)
    eager.use_graphs = False
    n = 300
    for r in (runner, eager):         # holds a slot and pages throughout, so the prompts below get other ones in turn
        r.add_request(100)
        r.step([StepEntry(100, tokens(20, vocab, 1), 0, [19])])
    for i in range(5):
        toks = tokens(n + 1, vocab, 70 + i)
        got = []
        for r in (runner, eager):
            r.add_request(i)
            a = r.step([StepEntry(i, toks[:n], 0, [n - 1])]).float().cpu().clone()
            b = r.step([StepEntry(i, toks[n:], n, [0])]).float().cpu().clone()
            if i < 4:
                r.free_request(i)
            got.append(torch.cat([a, b]))
        assert logit_err(got[0], got[1]) < 1e-3, (i, logit_err(got[0], got[1]))
    assert any(isinstance(k, tuple) and k[0] == "prompt" and g.graph is not None for k, g in runner._graphs.items())
    assert not eager._graphs


def test_decoding_with_a_token_s_keys_cut_into_parts(dirs, monkeypatch):
    """The same with the attention kernel made to cut the keys of decoded tokens into parts, as it does by itself only
    at contexts and chunk sizes beyond those of a quick test."""
    from util import force_chunked_decode
    force_chunked_decode(monkeypatch)
    d = dirs["B"]
    vocab = plain_config(d)["vocab"]
    reqs = {i: tokens(80, vocab, 50 + i) for i in range(2)}
    want = {i: oracle(d, t) for i, t in reqs.items()}
    runner = make_runner(d, "bfloat16", 256, 16, 4)
    got = run_schedule(runner, reqs, [[(0, 30), (1, 2)]] + [[(0, 1), (1, 1)]] * 50 + [[(1, 28)]])
    for i in reqs:
        assert_logits(got[i], want[i], "bfloat16", i)


def test_layers_without_a_feed_forward_and_checkpoint_sizes(tmp_path):
    """A model none of whose layers has a feed-forward, with low-rank sizes that only the checkpoint knows."""
    cfg = config([layer(mlp=None, left={"mask": {"size": 3}}), layer(mlp=None, right={"conv": 5})], width=32, vocab=50)
    d = write_model(str(tmp_path / "m"), cfg, 5)
    assert plain_weights(d)["l0.mix.right.a1"].shape[0] == 16
    toks = tokens(40, 50, 1)
    runner = make_runner(d, "float32", 64, 16, 2)
    got = run_schedule(runner, {0: toks}, [[(0, 3)], [(0, 30)], [(0, 1)], [(0, 6)]])[0]
    assert logit_err(got, oracle(d, toks)) < TOL["float32"]


# ---- through the engine ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine_and_its_scheduler(dirs, dtype):
    """Requests of unequal lengths through ``LlmEngine.generate``: continuous batching with prompts in portions (a token
    budget below the longest prompt) beside decoding requests, greedy tokens against the plain model."""
    from atoma_infer_amd.config.engine import CacheConfig, SchedulerConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling.params import GenerateParameters
    d = dirs["A"]
    cfg, w = plain_config(d), plain_weights(d)
    prompts = [tokens(n, cfg["vocab"], 60 + n) for n in (3, 41, 17, 1, 29)]
    eng = LlmEngine(d, dtype, cache=CacheConfig(block_size=16, num_gpu_blocks_override=24),
                    scheduler=SchedulerConfig(max_num_batched_tokens=24, max_num_sequences=4, max_model_len=128,
                                              enable_chunked_prefill=True))
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=12, ignore_eos_token=True))
    off = 0
    for p, o in zip(prompts, outs):
        got = o.inference_outputs[0].token_ids
        assert len(got) == 12
        rows = ps.forward(list(p) + got, w, cfg)[len(p) - 1: -1]
        for step, tok in enumerate(got):
            # the engine's token is the plain model's argmax, up to logits that rounding cannot tell apart
            gap = float(rows[step].max() - rows[step][tok])
            off += gap > (1e-4 if dtype == "float32" else 0.08) * float(rows[step].abs().max())
    # (bfloat16: a token that rounding sends to another expert than the plain model's may pick another token)
    assert off <= (0 if dtype == "float32" else 6), off


def test_the_trace_program_runs_the_design(dirs, tmp_path):
    import json
    import os
    import subprocess
    import sys
    d = dirs["A"]
    toks = tokens(30, plain_config(d)["vocab"], 8)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:9], "want": [0, 8]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[9:], "want": [20]},
                                     {"id": "y", "tokens": toks[:4], "want": [3]}], "end": ["x", "y"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "out")
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                           "--out", out, "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1"]
    want = oracle(d, toks)
    a = torch.from_numpy(np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(2, -1))
    b = torch.from_numpy(np.fromfile(os.path.join(out, "1.f32"), dtype="<f4").reshape(2, -1))
    assert logit_err(a, want[[0, 8]]) < TOL["float32"] and logit_err(b, want[[29, 3]]) < TOL["float32"]

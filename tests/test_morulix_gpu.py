"""Morulix on the GPU against the plain implementation: every mechanism alone, then the whole model through the
runner's step function (portions, batches, pages and slots used again) and through the engine's own entry point."""
import copy
import types

import numpy as np
import pytest
import torch

import plain_morulix as pm
from morulix_util import MOR_A, MOR_B, MOR_C, MOR_D, SCALING, attention, config, latent, layer, mamba
from somesun_util import logit_err, make_runner, plain_config, plain_weights, run_schedule, tokens, write_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# float32: the engine's sums run in another order than the plain model's float64 ones; bfloat16: activations are
# rounded to 8 bits about ten times a layer
TOL = {"float32": 3e-5, "bfloat16": 4e-2}
PART_TOL = {torch.float32: 2e-5, torch.bfloat16: 2.5e-2}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("morulix")
    return {n: write_model(str(root / n), c, 11 + i) for i, (n, c) in
            enumerate((("A", MOR_A), ("B", MOR_B), ("C", MOR_C), ("D", MOR_D)))}


def oracle(path, toks):
    return pm.forward(list(toks), plain_weights(path), plain_config(path)).float()


def assert_logits(got, want, dtype, what=""):
    """Every row's difference (row means taken off, root mean square over the vocabulary) against the spread of the
    request's logits as a whole: a row whose own logits happen to be small is not held to a smaller error."""
    d = got.double() - want.double()
    d = d - d.mean(dim=-1, keepdim=True)
    w = want.double() - want.double().mean(dim=-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()
    if dtype == "float32":
        assert float(e.max()) < TOL[dtype], (what, float(e.max()), int(e.argmax()))
        return
    # bfloat16: rounding's effect has a long tail (a few tokens of a random model sit where a gate or a softmax is
    # steep, and every path of the engine, like every order of rounding, is several times further off there than at the
    # median token), while a fault of a cache, a state or a mask puts its rows off by their whole size
    assert float(e.median()) < TOL[dtype] / 3 and float((e < TOL[dtype]).double().mean()) >= 0.95 \
        and float(e.max()) < 4 * TOL[dtype], (what, float(e.median()), float(e.max()), int(e.argmax()))


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


def _drawn(part, tag, seed, boost=()):
    """Random tensors for a part as bfloat16 values held in float32; ``boost`` names tensors to make larger."""
    from atoma_infer_amd.weights.random_init import random_tensor
    w = {n: random_tensor(tag + n, ws, seed, torch.bfloat16, 0.1).float() for n, ws in part.weight_specs().items()}
    for n, f in boost:
        w[n] = (w[n] * f).to(torch.bfloat16).float()
    return w


def _flat(y):
    return (y.sum(0) if y.dim() == 3 else y).float().cpu()


def _rel(a, b):
    return float((a.double() - b.double()).norm() / b.double().norm())


# ---- small kernels ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("width, planes", [(64, (1, 1)), (200, (2, 3)), (4100, (1, 0)), (50, (3, 1))])
def test_sublayer_outputs_join_the_stream_unnormed(width, planes):
    """The side-by-side block's sum: resid += a + b, and the next norm (weight 1 + w) of the new rows, one kernel."""
    from atoma_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(width)
    t = 5
    resid = torch.randn(t, width, generator=g)
    terms = [(torch.randn(planes[0], t, width, generator=g), 1.0)]
    if planes[1]:
        terms.append((torch.randn(planes[1], t, width, generator=g).to(torch.bfloat16), 1.0))
    wn = torch.randn(width, generator=g) * 0.1
    want_resid = resid.double() + sum(x.double().sum(0) * s for x, s in terms)
    want_out = pm.norm_around_zero(want_resid, wn.double(), 2e-6)
    dev_terms = [((x[0] if x.shape[0] == 1 else x).contiguous().to(DEV), s) for x, s in terms]
    for out_dtype in (torch.float32, torch.bfloat16):
        r = resid.to(DEV)
        out = ops.add_normed(r, dev_terms, None, 0.0, (1.0 + wn).to(DEV), 2e-6, out_dtype)
        assert (r.cpu().double() - want_resid).abs().max() < 2e-5
        assert (out.cpu().double() - want_out).abs().max() < (2e-5 if out_dtype is torch.float32 else 4e-2)
    r2 = resid.to(DEV)
    assert ops.add_normed(r2, dev_terms, None, 0.0) is None and torch.equal(r2, r)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, times", [(64, 2), (96, 1), (200, 3)])
def test_loop_entry_alone(width, times, dtype):
    from atoma_infer_amd.parts import LoopEntry
    part = LoopEntry(width, times)
    w = _drawn(part, "loop.", 2)
    _load(part, w, dtype)
    g = torch.Generator().manual_seed(times)
    x, e, d = (torch.randn(7, width, generator=g) for _ in range(3))
    for turn in range(times):
        resid = x.to(DEV)
        assert part.forward(resid, d.to(DEV), None, None, embedded=e.to(DEV), turn=turn) is None
        want = torch.cat([x.double() + d.double(), e.double()], -1) @ w["in"].double().T + w["step"][turn].double()
        assert _rel(resid.cpu(), want) < (2e-6 if dtype is torch.float32 else 8e-3)
    with pytest.raises(RuntimeError):
        part.forward(x.to(DEV), None, None, None, embedded=e.to(DEV), turn=times)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t, h, k, n", [(1, 1, 8, 8), (5, 3, 24, 20), (70, 8, 64, 48), (33, 2, 100, 130), (17, 5, 7, 3)])
def test_a_product_of_its_own_per_head(t, h, k, n, dtype):
    from atoma_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(t + n)
    x = torch.randn(t, h * k, generator=g).to(torch.bfloat16).float()
    w = torch.randn(h, n, k, generator=g).to(torch.bfloat16).float()
    gate = torch.rand(t, h, generator=g)
    want = torch.einsum("thk,hnk->thn", x.view(t, h, k).double(), w.double())
    got = ops.head_linear(x.to(DEV, dtype), w.to(DEV, torch.bfloat16), dtype)
    assert _rel(got.float().cpu().view(t, h, n), want) < (1e-6 if dtype is torch.float32 else 5e-3)
    got = ops.head_linear(x.to(DEV, dtype), w.to(DEV, torch.bfloat16), dtype, gate.to(DEV))
    assert _rel(got.float().cpu().view(t, h, n), want * gate.double()[:, :, None]) < (1e-6 if dtype is torch.float32 else 5e-3)
    # rows of a wider tensor
    wide = torch.zeros(t, h * k + 16, dtype=dtype, device=DEV)
    wide[:, : h * k] = x.to(DEV, dtype)
    assert torch.equal(ops.head_linear(wide[:, : h * k], w.to(DEV, torch.bfloat16), dtype, gate.to(DEV)), got)


# ---- the recurrence alone ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, groups, vdim, n, taps, parts", [(4, 2, 16, 16, 3, 2), (3, 1, 8, 12, 2, 1), (2, 2, 40, 100, 5, 5),
                                                                 (1, 1, 5, 1, 1, 5), (6, 3, 24, 200, 4, 3), (4, 4, 64, 48, 4, 2),
                                                                 (2, 1, 32, 128, 4, 1), (1, 1, 4200, 4, 2, 1)])
def test_state_space_recurrence_alone_whole_and_in_portions(heads, groups, vdim, n, taps, parts, dtype):
    """The mixer on hand-made steps: two requests side by side, cut into portions of unequal lengths (one token, two,
    fewer than the convolution has taps, many), each carried by its state slot; against the plain recurrence.  Portions
    of 16 tokens and more run 64 tokens at a time on the matrix cores (states up to 128), shorter ones token by token:
    the portions here are of both kinds, side by side in one step too, with chunks that are full and that are not."""
    from atoma_infer_amd.parts import StateSpaceDuality
    width = 64
    part = StateSpaceDuality(width, heads, groups, vdim, n, taps, parts, 1e-5)
    w = _drawn(part, "x.", 5, boost=(("in", 8),))
    _load(part, w, dtype)
    g = torch.Generator().manual_seed(n)
    lens = (267, 29)
    hs = [torch.randn(c, width, generator=g).to(torch.bfloat16).float() for c in lens]
    m = {"heads": heads, "groups": groups, "vdim": vdim, "state": n, "conv": taps, "norm_groups": parts}
    want = [pm.mamba2(h.double(), {"r." + k: v.double() for k, v in w.items()}, "r.", m, 1e-5) for h in hs]
    state = torch.zeros((4, part.state_spec().shape[0]), dtype=torch.float32, device=DEV)
    state[1].fill_(7.0)                       # another request's slot must stay as it is
    cache = types.SimpleNamespace(state=state)
    got, at = [[], []], [0, 0]
    for cuts in ([(0, 1), (1, 2)], [(0, 2)], [(1, 1), (0, 1)], [(0, 30), (1, 6)], [(0, 3)], [(0, 64), (1, 17)], [(0, 150)],
                 [(0, 16), (1, 3)]):
        ctx = _ctx([at[r] for r, _ in cuts], [c for _, c in cuts], [3 if r == 0 else 0 for r, _ in cuts])
        x = torch.cat([hs[r][at[r]: at[r] + c] for r, c in cuts]).to(DEV, dtype)
        y = _flat(part.forward(x, ctx, cache))
        o = 0
        for r, c in cuts:
            got[r].append(y[o: o + c])
            o += c
            at[r] += c
    assert at == list(lens) and bool((state[1] == 7.0).all())
    for r in range(2):
        assert _rel(torch.cat(got[r]), want[r]) < PART_TOL[dtype], r


def test_a_far_token_stays_in_the_recurrent_state():
    """Decays close to one and one early token whose input is large: hundreds of tokens later the read-out still holds
    it.  A state that is lost, cleared or carried by the wrong slot changes the late outputs entirely."""
    from atoma_infer_amd.parts import StateSpaceDuality
    width, heads, vdim, n, taps = 64, 2, 16, 32, 2
    part = StateSpaceDuality(width, heads, 1, vdim, n, taps, 1, 1e-5)
    w = _drawn(part, "y.", 9, boost=(("in", 4),))
    w["A_log"] = torch.full_like(w["A_log"], -7.0)             # exp(-exp(-7) dt): the state hardly decays
    w["D"] = w["D"] * 0
    _load(part, w, torch.float32)
    g = torch.Generator().manual_seed(1)
    count = 400
    h = torch.randn(count, width, generator=g).to(torch.bfloat16).float() * 0.3
    h[5] = h[5] * 40                                            # the far token
    m = {"heads": heads, "groups": 1, "vdim": vdim, "state": n, "conv": taps, "norm_groups": 1}
    pw = {"r." + k: v.double() for k, v in w.items()}
    want = pm.mamba2(h.double(), pw, "r.", m, 1e-5)
    h_without = h.clone()
    h_without[5] = h[5] / 40
    assert (pm.mamba2(h_without.double(), pw, "r.", m, 1e-5)[-20:] - want[-20:]).norm() > 0.2 * want[-20:].norm()
    state = torch.zeros((2, part.state_spec().shape[0]), dtype=torch.float32, device=DEV)
    cache = types.SimpleNamespace(state=state)
    got, at = [], 0
    for c in [300, 63, 2] + [1] * 35:
        got.append(_flat(part.forward(h[at: at + c].to(DEV), _ctx([at], [c], [1]), cache)))
        at += c
    got = torch.cat(got)
    assert _rel(got, want) < 2e-5 and _rel(got[-20:], want[-20:]) < 2e-5


# ---- the two kinds of attention alone -------------------------------------------------------------------------------

def _paged_case(part, plain, dtype, lens_and_cuts, page, seed, boost=None, width=64):
    """A mixer with a paged cache on hand-made steps over pages that are dealt out of order: per request the outputs
    of all its portions, and the plain function's on the whole request."""
    lens = [sum(c for r2, c in sum(lens_and_cuts, []) if r2 == r) for r in range(2)]
    g = torch.Generator().manual_seed(seed)
    hs = [torch.randn(c, width, generator=g).to(torch.bfloat16).float() for c in lens]
    if boost is not None:
        # one position whose key every later query of the request scores far above all others, if it may see it
        r, p = boost
        hs[r][p + 1:] = (hs[r][p + 1:] * 0.2 + hs[r][p] * 3).to(torch.bfloat16).float()
    want = [plain(h.double()) for h in hs if len(h)]
    cs = part.cache_spec()
    n_pages = sum(-(-c // page) for c in lens) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    tables = [[order.pop() for _ in range(-(-c // page))] for c in lens]
    max_blocks = max(len(tb) for tb in tables)
    k = torch.zeros((n_pages, cs.kv_heads, page * cs.head_size), dtype=dtype, device=DEV)
    v = torch.zeros_like(k)
    got, at = [[], []], [0, 0]
    for cuts in lens_and_cuts:
        ctx = _ctx([at[r] for r, _ in cuts], [c for _, c in cuts], [0] * len(cuts))
        bt = torch.tensor([tables[r] + [0] * (max_blocks - len(tables[r])) for r, _ in cuts], dtype=torch.int32, device=DEV)
        slots = [tables[r][(at[r] + j) // page] * page + (at[r] + j) % page for r, c in cuts for j in range(c)]
        cache = types.SimpleNamespace(k=k, v=v, page_size=page, writable=True, block_tables=bt,
                                      slot_mapping=torch.tensor(slots, dtype=torch.int32, device=DEV))
        x = torch.cat([hs[r][at[r]: at[r] + c] for r, c in cuts]).to(DEV, dtype)
        y = _flat(part.forward(x, ctx, cache))
        o = 0
        for r, c in cuts:
            got[r].append(y[o: o + c])
            o += c
            at[r] += c
    return [torch.cat(x) for x in got if x], want


CUTS = [[(0, 20), (1, 3)], [(0, 1), (1, 1)], [(0, 2)], [(1, 40), (0, 1)], [(0, 50)], [(0, 1)], [(1, 1)], [(0, 1), (1, 2)]]


def _window_part(m, dtype, seed=7, width=64):
    from atoma_infer_amd.parts import PagedAttention, RotaryEncoding
    position = None
    if m.get("rot"):
        sc = m["rot"].get("scaling")
        sc = None if sc is None else {"factor": sc["factor"], "low_freq_factor": sc["low"], "high_freq_factor": sc["high"],
                                      "original_max_position_embeddings": sc["original"]}
        position = RotaryEncoding(m["dim"], m["rot"]["base"], 2048, sc, m["rot"]["dims"], precise=True)
    part = PagedAttention(width, m["heads"], m["kv_heads"], m["dim"], position, m["mask"]["size"] if m.get("mask") else None,
                          m["scale"], value_size=m["vdim"], names=("q", "k", "v", "o"))
    w = _drawn(part, "t.", seed, boost=(("q", 30), ("k", 30), ("v", 10), ("o", 5)))
    _load(part, w, dtype)
    pw = {"a." + k: v.double() for k, v in w.items()}
    return part, lambda h: pm.windowed_attention(h, pw, "a.", m)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m, page", [
    (attention(dim=32, heads=4, kv_heads=2, vdim=16, scale=0.3, window=5, rot_dims=8, base=100.0, scaling=SCALING), 16),
    (attention(dim=64, heads=8, kv_heads=2, scale=0.1, window=33, rot_dims=64, base=500.0), 16),
    (attention(dim=40, heads=6, kv_heads=3, vdim=48, scale=0.16, window=100, rot_dims=20, base=30.0), 32),
    (attention(dim=16, heads=1, kv_heads=1, scale=1.0, window=1, rot_dims=2, base=2.0), 16),
    (attention(dim=64, heads=4, kv_heads=1, vdim=32, scale=0.11, window=None, rot_dims=None), 16),
    (attention(dim=24, heads=3, kv_heads=1, vdim=24, scale=0.2, window=16, rot_dims=24, base=77.0), 4),
])
def test_windowed_attention_alone(m, page, dtype):
    """Values narrower and wider than the keys; part of a head rotated, all of it, none; windows of one key, of a page
    and a bit, longer than the requests, none; pages of 4, 16 and 32 tokens."""
    part, plain = _window_part(m, dtype)
    got, want = _paged_case(part, plain, dtype, CUTS, page, seed=m["dim"])
    for a, b in zip(got, want):
        assert _rel(a, b) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("edge", [0, 1])
def test_a_dominant_key_just_inside_and_just_outside_the_window(dtype, edge):
    """A key that outweighs all others: the token ``window - 1`` positions later still sees it, the next one does not,
    in a prompt's portion and token by token.  A window that is one position off changes those rows entirely."""
    window, p = 24, 29
    m = attention(dim=64, heads=4, kv_heads=1, scale=0.6, window=window, rot_dims=16, base=50.0)
    part, plain = _window_part(m, dtype)
    # the position p + window - 1 + edge is the last of a prompt's portion in one request and decoded alone in the other
    last = p + window - 1 + edge
    cuts = [[(0, 30), (1, 30)], [(0, last - 30 + 1), (1, last - 30 - 3)]] + [[(1, 1)]] * 8 + [[(0, 2)], [(0, 1)]]
    got, want = _paged_case(part, plain, dtype, cuts, 16, seed=3, boost=(0, p))
    got1, want1 = _paged_case(part, plain, dtype, cuts, 16, seed=3, boost=(1, p))
    for a, b in ((got[0], want[0]), (got1[1], want1[1])):
        rows = slice(p + window - 3, p + window + 2)
        assert _rel(a[rows], b[rows]) < PART_TOL[dtype] and _rel(a, b) < PART_TOL[dtype]
    # the plain rows on the two sides of the edge do differ: the test can see a window that is off by one
    assert _rel(want[0][p + window - 1], want[0][p + window]) > 0.3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [300, None])
def test_a_far_key_under_a_long_window_and_behind_it(dtype, window):
    """A dominant key hundreds of positions back, at a page's last slot: under a window of 300 keys the rows up to 299
    positions later are made of its value and the rows behind are not; without a window every later row is.  Rows in a
    long portion, in portions of two tokens and decoded alone stand on both sides of the edge."""
    p = 31
    # (a few columns rotated: the others carry the key's weight over any distance)
    m = attention(dim=64, heads=4, kv_heads=2, vdim=32, scale=0.6, window=window, rot_dims=8, base=200.0)
    part, plain = _window_part(m, dtype)
    edge = p + 300                      # the first position that no longer sees the key under the window
    cuts = [[(0, 200), (1, 5)], [(0, edge - 200 - 3)], [(0, 2)], [(0, 1)], [(0, 1)], [(0, 2)], [(0, 1)], [(0, 40), (1, 1)]] + \
        [[(0, 1)]] * 6
    got, want = _paged_case(part, plain, dtype, cuts, 16, seed=9, boost=(0, p))
    rows = slice(edge - 4, edge + 4)
    assert _rel(got[0][rows], want[0][rows]) < PART_TOL[dtype] and _rel(got[0], want[0]) < PART_TOL[dtype]
    far = _rel(want[0][edge - 1], want[0][edge])
    assert far > 0.3 if window else far < 0.3        # (the plain rows say whether there is an edge to see)


def _latent_part(m, dtype, seed=7, width=64, sink_value=None):
    from atoma_infer_amd.parts import LatentAttention
    part = LatentAttention(width, m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["scale"], 1e-5)
    w = _drawn(part, "l.", seed, boost=(("q", 30), ("dkv", 10), ("uv", 3), ("o", 5), ("g", 10)))
    if sink_value is not None:
        w["sink"] = torch.full_like(w["sink"], sink_value)
    _load(part, w, dtype)
    pw = {"a." + k: v.double() for k, v in w.items()}
    return part, lambda h: pm.latent_attention(h, pw, "a.", m, 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m, page", [(latent(dim=32, heads=4, vdim=24, kv_rank=16, scale=0.2), 16),
                                     (latent(dim=24, heads=3, vdim=40, kv_rank=20, scale=0.25), 16),
                                     (latent(dim=32, heads=8, vdim=32, kv_rank=48, scale=0.18), 32),
                                     (latent(dim=8, heads=1, vdim=8, kv_rank=8, scale=0.5), 16),
                                     (latent(dim=48, heads=2, vdim=16, kv_rank=64, scale=0.15), 4),
                                     (latent(dim=16, heads=12, vdim=8, kv_rank=128, scale=0.1), 16)])
def test_latent_attention_alone(m, page, dtype):
    """Latents narrower and wider than the heads' keys, sizes that are no multiple of 16, one head and twelve; only the
    latent is cached, the heads' key and value maps act on the queries and on the mixed latents."""
    part, plain = _latent_part(m, dtype)
    assert part.cache_spec().kv_heads == 1 and part.cache_spec().head_size == -(-m["kv_rank"] // 16) * 16
    got, want = _paged_case(part, plain, dtype, CUTS, page, seed=m["dim"])
    for a, b in zip(got, want):
        assert _rel(a, b) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sink", [-30.0, 0.0, 6.0])
def test_the_sink_takes_its_share(sink, dtype):
    """A sink far below the scores changes nothing, one far above takes nearly all of the weight."""
    m = latent(dim=32, heads=4, vdim=24, kv_rank=32, scale=0.2)
    part, plain = _latent_part(m, dtype, sink_value=sink)
    got, want = _paged_case(part, plain, dtype, CUTS, 16, seed=1)
    for a, b in zip(got, want):
        assert _rel(a, b) < PART_TOL[dtype]
    if sink != 0.0:
        part0, _ = _latent_part(m, dtype, sink_value=0.0)
        zero, _ = _paged_case(part0, plain, dtype, CUTS, 16, seed=1)
        assert (got[0] - zero[0]).norm() > 0.05 * zero[0].norm()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds(dtype):
    """One early key that outweighs the hundreds behind it, at a page's last slot: every later row, in long portions, in
    short ones and decoded alone, is made of that key's value."""
    m = latent(dim=32, heads=4, vdim=24, kv_rank=32, scale=0.5)
    part, plain = _latent_part(m, dtype, sink_value=-5.0)
    cuts = [[(0, 100), (1, 7)], [(0, 500)], [(0, 2), (1, 1)], [(0, 38)]] + [[(0, 1)]] * 12
    got, want = _paged_case(part, plain, dtype, cuts, 16, seed=5, boost=(0, 15))
    assert _rel(got[0], want[0]) < PART_TOL[dtype] and _rel(got[0][-14:], want[0][-14:]) < PART_TOL[dtype]


# ---- the whole model through the step function --------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_prompts_token_by_token_decoding_and_portions(dirs, name, dtype):
    d = dirs[name]
    vocab = plain_config(d)["vocab"]
    toks = tokens(150, vocab, 3)
    want = oracle(d, toks)
    runner = make_runner(d, dtype, 256, 16, 4)
    n = len(toks)
    schedules = {
        "whole": [[(0, n)]],
        "tokens": [[(0, 1)]] * n,                                        # crosses every window and page edge one token at a time
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
@pytest.mark.parametrize("name", ["A", "B", "D"])
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
    recurrent state, the convolution's inputs and the loop's passes are read from the step's device tensors."""
    d = dirs["B"]
    vocab = plain_config(d)["vocab"]
    reqs = {i: tokens(60, vocab, 40 + i) for i in range(3)}
    want = {i: oracle(d, t) for i, t in reqs.items()}
    sched = [[(0, 20), (1, 5), (2, 9)]] + [[(0, 1), (1, 1), (2, 1)]] * 40 + [[(1, 15)], [(2, 11)]]
    for name in ("B", "A"):
        d = dirs[name]
        vocab = plain_config(d)["vocab"]
        reqs = {i: tokens(60, vocab, 40 + i) for i in range(3)}
        want = {i: oracle(d, t) for i, t in reqs.items()}
        runner = make_runner(d, "bfloat16", 256, 16, 4)
        assert runner.use_graphs
        got = run_schedule(runner, reqs, sched)
        assert any(g.graph is not None for g in runner._graphs.values())
        for i in reqs:
            assert_logits(got[i], want[i], "bfloat16", (name, i))


def test_a_lone_prompt_s_step_replayed_as_a_graph(dirs):
    """A step that is one prompt of 256 tokens or more and wants its last place is recorded the third time its shape is
    seen: every replay, with other tokens and another state slot, gives what a runner without graphs gives."""
    from atoma_infer_amd.engine.step import StepEntry
    d = dirs["D"]
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


def test_a_layer_order_of_its_own_and_pages_of_other_sizes(tmp_path):
    """The same kind of mixer twice in a row, the recurrence last, a loop in the middle that runs four times, widths that
    are no multiple of 32, pages of 32 and 48 tokens."""
    cfg = config([layer("attention", attention(dim=16, heads=2, kv_heads=2, scale=0.25, window=9, rot_dims=16, base=10.0), ff=24),
                  layer("attention", attention(dim=16, heads=2, kv_heads=1, scale=0.25, window=20, rot_dims=4, base=10.0), ff=None),
                  layer("latent_attention", latent(dim=16, heads=2, vdim=16, kv_rank=24, scale=0.3), ff=None),
                  layer("mamba2", mamba(heads=2, groups=2, vdim=12, state=8, conv=3, norm_groups=3), ff=20)],
                 width=40, vocab=60, loop=(1, 3, 4))
    d = write_model(str(tmp_path / "m"), cfg, 5)
    toks = tokens(70, 60, 1)
    want = oracle(d, toks)
    for dtype, page in (("float32", 32), ("bfloat16", 48), ("bfloat16", 32)):
        runner = make_runner(d, dtype, 192, page, 2)
        got = run_schedule(runner, {0: toks}, [[(0, 3)], [(0, 30)], [(0, 1)], [(0, 2)], [(0, 33)], [(0, 1)]])[0]
        assert_logits(got, want, dtype, (dtype, page))


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
        rows = pm.forward(list(p) + got, w, cfg)[len(p) - 1: -1]
        for step, tok in enumerate(got):
            # the engine's token is the plain model's argmax, up to logits that rounding cannot tell apart
            gap = float(rows[step].max() - rows[step][tok])
            off += gap > (1e-4 if dtype == "float32" else 0.08) * float(rows[step].abs().max())
    assert off == 0, off


def test_the_trace_program_runs_the_design(dirs, tmp_path):
    import json
    import os
    import subprocess
    import sys
    d = dirs["D"]
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

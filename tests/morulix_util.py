"""Shared pieces of the Morulix tests: small configurations that differ from each other in every size."""
from __future__ import annotations


def attention(dim=32, heads=4, kv_heads=2, vdim=None, scale=0.2, window=7, rot_dims=16, base=1000.0, scaling=None):
    m = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": dim if vdim is None else vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if rot_dims is not None:
        m["rot"] = {"base": base, "dims": rot_dims}
        if scaling is not None:
            m["rot"]["scaling"] = scaling
    return m


def latent(dim=32, heads=4, vdim=24, kv_rank=16, scale=0.2):
    return {"dim": dim, "heads": heads, "kv_rank": kv_rank, "scale": scale, "vdim": vdim}


def mamba(heads=4, groups=2, vdim=16, state=16, conv=3, norm_groups=2):
    return {"conv": conv, "groups": groups, "heads": heads, "norm_groups": norm_groups, "state": state, "vdim": vdim}


def layer(kind, mixer, ff=48):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=64, vocab=97, eps=1e-5, loop=None):
    c = {"architecture": "Morulix", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop is not None:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


SCALING = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}

# the recurrence first, then a window of five keys with part of the head rotated and values half as wide as the keys,
# then a latent of 20 numbers (no multiple of 16) with values wider than the keys; the last two layers run three
# times; one layer has no feed-forward; a state size and a head width that are no multiples of anything
MOR_A = config([
    layer("mamba2", mamba(heads=3, groups=1, vdim=8, state=12, conv=2, norm_groups=1), ff=40),
    layer("attention", attention(dim=32, heads=4, kv_heads=2, vdim=16, scale=0.3, window=5, rot_dims=8, base=100.0,
                                 scaling=SCALING), ff=None),
    layer("latent_attention", latent(dim=24, heads=3, vdim=40, kv_rank=20, scale=0.25), ff=56),
], width=64, vocab=97, loop=(1, 3, 3))
# no loop at all; heads of 64 columns (the matrix-core attention in bfloat16); a window that is no multiple of a page,
# the whole head rotated without rescaling; every head its own B and C; an attention layer that sees all keys with
# one shared key head and no rotation
MOR_B = config([
    layer("latent_attention", latent(dim=32, heads=8, vdim=32, kv_rank=48, scale=0.18), ff=96),
    layer("attention", attention(dim=64, heads=8, kv_heads=8, scale=0.125, window=33, rot_dims=64, base=500.0), ff=64),
    layer("mamba2", mamba(heads=4, groups=4, vdim=32, state=64, conv=4, norm_groups=4), ff=32),
    layer("attention", attention(dim=64, heads=4, kv_heads=1, vdim=32, scale=0.11, window=None, rot_dims=None), ff=64),
], width=128, vocab=211, eps=3e-6)
# everything that can be one is one: a loop of one pass over all layers, one head, one group, one key head, a window
# of one key, a norm group per column, a convolution of one tap
MOR_C = config([
    layer("attention", attention(dim=16, heads=1, kv_heads=1, scale=1.0, window=1, rot_dims=2, base=2.0), ff=16),
    layer("mamba2", mamba(heads=1, groups=1, vdim=16, state=1, conv=1, norm_groups=16), ff=None),
    layer("latent_attention", latent(dim=8, heads=1, vdim=8, kv_rank=8, scale=0.5), ff=24),
], width=32, vocab=50, loop=(0, 3, 1))
# a loop over the first layers only, twice, with a window longer than most requests and a state wider than a
# workgroup's lanes hold in one register each
MOR_D = config([
    layer("latent_attention", latent(dim=48, heads=2, vdim=16, kv_rank=64, scale=0.15), ff=64),
    layer("mamba2", mamba(heads=2, groups=1, vdim=40, state=100, conv=5, norm_groups=5), ff=64),
    layer("attention", attention(dim=40, heads=6, kv_heads=3, vdim=48, scale=0.16, window=100, rot_dims=20, base=30.0,
                                 scaling={"factor": 3.0, "low": 0.5, "high": 2.0, "original": 40}), ff=64),
], width=96, vocab=130, loop=(0, 2, 2))

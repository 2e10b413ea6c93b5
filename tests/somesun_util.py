"""Shared pieces of the Somesun tests: small configurations, model folders, runs through the runner."""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Sequence, Tuple

import torch


def layer(left=None, right=None, mlp="default", left_scale=0.7, right_scale=1.3):
    """A layer entry of config.json; the arguments overwrite the defaults key by key (``mlp=None``: no feed-forward)."""
    l = {"dim": 32, "heads": 4, "kv_heads": 2, "vdim": 32, "scale": 0.2, "mask": {"size": 7},
         "rot": {"base": 1000.0, "dims": 16}}
    r = {"dim": 16, "heads": 4, "kv_heads": 2, "vdim": 24, "conv": 3}
    m = {"kind": "moe", "expert": {"ff": 48}, "router": {"experts": 4, "top": 2}}
    l.update(left or {})
    if "vdim" not in (left or {}):
        l["vdim"] = l["dim"]
    r.update(right or {})
    if mlp is None:
        m = None
    elif mlp != "default":
        m = {"kind": "moe", "expert": {"ff": mlp["ff"]}, "router": {"experts": mlp["experts"], "top": mlp["top"]}}
    return {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": m}


def config(layers, width=64, vocab=97, eps=1e-5):
    return {"architecture": "Somesun", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


# Two layers that differ in every size: grouped and shared key heads, part of a head rotated against all of it,
# chunks of 7 and of 16 positions, grouped q/k heads in the recurrence against one each, a key size that is no multiple
# of 8, 3 and 4 taps, two of four experts against no feed-forward at all, low-rank sizes named against the checkpoint's.
SUN_A = config([
    layer(right={"decay_rank": 5, "gate_rank": 6}),
    layer(left={"dim": 48, "heads": 2, "kv_heads": 1, "scale": 0.11, "mask": {"size": 16}, "rot": {"base": 50.0, "dims": 48}},
          right={"dim": 40, "heads": 2, "kv_heads": 2, "vdim": 8, "conv": 4}, mlp=None, left_scale=1.0, right_scale=0.4),
])
# Heads of 64 columns (the matrix-core attention in bfloat16), chunks of 33, one expert of three, one tap less, a
# recurrence with one q/k head for three heads of wide values, another eps
SUN_B = config([
    layer(left={"dim": 64, "heads": 8, "kv_heads": 2, "scale": 0.08, "mask": {"size": 33}, "rot": {"base": 500.0, "dims": 32}},
          right={"dim": 64, "heads": 3, "kv_heads": 1, "vdim": 40, "conv": 2},
          mlp={"ff": 64, "experts": 3, "top": 1}, left_scale=0.5, right_scale=0.5),
    layer(left={"dim": 64, "heads": 4, "kv_heads": 4, "scale": 0.125, "mask": {"size": 33}, "rot": {"base": 500.0, "dims": 64}},
          right={"dim": 128, "heads": 2, "kv_heads": 2, "vdim": 16, "conv": 1},
          mlp={"ff": 32, "experts": 5, "top": 3}),
], width=128, vocab=211, eps=3e-6)
# head sizes that the matrix-core attention does not take as they are (36 and 40: run as 48)
SUN_C = config([
    layer(left={"dim": 36, "heads": 2, "kv_heads": 1, "scale": 0.2, "mask": {"size": 11}, "rot": {"base": 77.0, "dims": 18}},
          right={"dim": 24, "heads": 2, "kv_heads": 1, "vdim": 12, "conv": 2}, mlp={"ff": 32, "experts": 2, "top": 2}),
    layer(left={"dim": 40, "heads": 3, "kv_heads": 3, "scale": 0.15, "mask": {"size": 64}, "rot": {"base": 77.0, "dims": 40}},
          right={"dim": 8, "heads": 1, "kv_heads": 1, "vdim": 64, "conv": 3}, mlp={"ff": 40, "experts": 6, "top": 1}),
], width=96, vocab=130)


def write_model(path: str, cfg: dict, seed: int, changes=None) -> str:
    """A model folder with random weights; ``changes(tensors)`` may overwrite tensors (float32 in, stored bfloat16)."""
    from atoma_infer_amd.weights import write_random_model
    write_random_model(path, copy.deepcopy(cfg), seed=seed, dtype="bfloat16", norm_jitter=0.1)
    if changes is not None:
        from safetensors.torch import load_file, save_file
        f = os.path.join(path, "model.safetensors")
        tensors = {k: v.to(torch.float32) for k, v in load_file(f).items()}
        changes(tensors)
        save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()}, f)
    return path


def plain_weights(path: str, dtype=torch.float64) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file
    return {k: v.to(dtype) for k, v in load_file(os.path.join(path, "model.safetensors")).items()}


def plain_config(path: str) -> dict:
    with open(os.path.join(path, "config.json")) as f:
        return json.load(f)


def make_runner(path: str, dtype: str, max_tokens: int, page_size: int = 16, slots: int = 4):
    from atoma_infer_amd.engine.replay import make_runner as mk
    return mk(path, dtype, max_tokens, page_size, slots)


def run_schedule(runner, requests: Dict[int, Sequence[int]], schedule: Sequence[Sequence[Tuple[int, int]]],
                 free: bool = True) -> Dict[int, torch.Tensor]:
    """Feed the requests' tokens through ``runner`` as ``schedule`` says (a list of steps, each a list of
    (request, tokens it brings)), asking for every position's logits; a request is admitted at its first entry and
    given back after its last token.  Returns request -> logits [tokens, vocab] on the CPU."""
    from atoma_infer_amd.engine.step import StepEntry
    at = {r: 0 for r in requests}
    rows: Dict[int, List[torch.Tensor]] = {r: [] for r in requests}
    for step in schedule:
        entries = []
        for r, n in step:
            if not runner.has_request(r):
                runner.add_request(r)
            entries.append(StepEntry(r, list(requests[r][at[r]: at[r] + n]), at[r], list(range(n))))
        logits = runner.step(entries).float().cpu()
        o = 0
        for r, n in step:
            rows[r].append(logits[o: o + n].clone())
            o += n
            at[r] += n
            if free and at[r] == len(requests[r]):
                runner.free_request(r)
    return {r: torch.cat(v) for r, v in rows.items() if v}


def tokens(n: int, vocab: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row: root mean square of the difference (row means taken off) over that of the wanted row."""
    d = got.double() - want.double()
    d = d - d.mean(dim=-1, keepdim=True)
    w = want.double() - want.double().mean(dim=-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-30)


def logit_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """The largest row error."""
    return float(row_errors(got, want).max())


def assert_logits(got: torch.Tensor, want: torch.Tensor, dtype: str, what="") -> None:
    """float32: every row within the tolerance.  bfloat16: rounding moves a router's scores by about a hundredth of
    their spread, so now and then a token of random weights goes to another expert than in the plain model, and its
    row and what later tokens make of it differ by more than rounding: half of the rows must be within half of the
    tolerance and nine in ten within it, which no fault of a cache, a state or a mask passes."""
    e = row_errors(got, want)
    if dtype == "float32":
        assert float(e.max()) < TOL[dtype], (what, float(e.max()), int(e.argmax()))
    else:
        assert float(e.median()) < TOL[dtype] / 2 and float((e < TOL[dtype]).double().mean()) >= 0.9, \
            (what, float(e.median()), float((e < TOL[dtype]).double().mean()))


# float32: the engine's sums run in another order than the plain model's float64 ones; bfloat16: activations are
# rounded to 8 bits about ten times a layer
TOL = {"float32": 3e-5, "bfloat16": 4e-2}

"""Small Vivisun configurations for the tests, their random weights, and the comparison with the plain decoder.

The configurations differ from one another in every size and option: heads of several sizes with keys and values of
different widths, one, several or all query heads to a key head, convolutions of one to five taps and none, rotations
over none, part or all of a head with and without bent frequencies, latent vectors narrower and wider than the heads
they feed, one head and many, layers without a feed-forward, stretches of layers that run once, twice and three times
from the first layer, the middle or to the last, sizes that are multiples of nothing.
"""
from __future__ import annotations

import os
from typing import Dict, List

import torch

from llm_rs_amd import VivisunConfig, random_model_tensors, write_model_folder
from plain_vivisun import bf16_rounding, plain_vivisun_logits


def dense(ff):
    return {"kind": "dense", "ff": ff}


def attention(heads, kv_heads, dim, vdim, scale, conv=0, rot_dims=None, base=10000.0, scaling=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "conv": conv,
         "rot": None if rot_dims is None else {"dims": rot_dims, "base": base, "scaling": scaling}}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent(heads, dim, vdim, kv_rank, scale, mlp=None):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale}, "mlp": mlp}


def config(width, vocab, layers, loop=None, eps=1e-5):
    return {"architecture": "Vivisun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
            "loop": None if loop is None else {"start": loop[0], "stop": loop[1], "times": loop[2]}}


BENT = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 2.0}

ODD = config(46, 97, [
    attention(6, 2, 10, 6, 0.3, conv=3, rot_dims=6, base=100.0, scaling=BENT, mlp=dense(30)),
    latent(3, 5, 7, 9, 0.4, mlp=dense(11)),
    attention(2, 2, 12, 20, 0.7, conv=1, rot_dims=12),
    latent(1, 13, 4, 17, 0.2, mlp=dense(17)),
], loop=(1, 3, 3))
PLAIN = config(64, 128, [
    latent(4, 16, 16, 32, 0.25, mlp=dense(96)),
    attention(4, 1, 16, 16, 0.25, conv=4, rot_dims=8, mlp=dense(32)),
    attention(2, 2, 32, 32, 0.2, conv=0, rot_dims=None, mlp=dense(64)),
], eps=1e-6)
# widths at which the bfloat16 products go to the matrix cores, heads and latent widths the matrix-core attention takes
WIDE = config(256, 320, [
    attention(8, 2, 64, 64, 0.125, conv=4, rot_dims=32, base=500.0, scaling=BENT, mlp=dense(512)),
    latent(8, 32, 32, 64, 0.2, mlp=dense(256)),
    latent(16, 64, 32, 128, 0.1),
    attention(4, 4, 32, 96, 0.2, conv=2, rot_dims=32, mlp=dense(128)),
], loop=(0, 2, 2))
CONFIGS = {"odd": ODD, "plain": PLAIN, "wide": WIDE}
PAGE_SIZE = {"odd": 4, "plain": 16, "wide": 16}


def one_layer(layer, width=40, vocab=61, loop=None):
    return config(width, vocab, [layer], loop)


def loud(tensors) -> None:
    """Random weights under which tokens differ: a dynamic tanh does not bring small embeddings up to size as a norm that
    divides would (its bias would be all that the layers see), so the token table is of order one; queries and the
    mixers' outputs are enlarged so that scores spread and what a mixer says counts beside the stream."""
    for name in list(tensors):
        factor = 50.0 if name == "embed" else 8.0 if name.endswith(".mix.q") else 4.0 if name.endswith(".mix.o") else None
        if factor is not None:
            tensors[name] = (tensors[name].double() * factor).to(tensors[name].dtype)


def make_model(cfg: dict, seed: int = 0, change=None):
    """(typed config, {name: bfloat16 tensor}); `change(tensors)` may put values of its own in."""
    typed = VivisunConfig.from_dict(cfg)
    tensors = random_model_tensors(typed, seed)
    loud(tensors)
    if change is not None:
        change(tensors)
    return typed, tensors


def make_folder(tmp_path, cfg: dict, seed: int = 0, change=None, name: str = "model") -> str:
    typed, tensors = make_model(cfg, seed, change)
    folder = os.path.join(str(tmp_path), name)
    write_model_folder(folder, typed, tensors)
    return folder


def reference(cfg: dict, tensors, requests: Dict[str, List[int]], rnd=None):
    kw = {} if rnd is None else {"rnd": rnd}
    return {rid: plain_vivisun_logits(cfg, tensors, toks, **kw) for rid, toks in requests.items()}


def allowed_error(dtype: str, cfg: dict, tensors, requests, exact) -> float:
    """How far the engine may be from the exact logits, as a part of a sequence's largest logit.  float32: 3e-5.
    bfloat16: twice as far as the plain decoder gets when every activation that passes through memory between two
    stages is rounded to bfloat16 (the engine keeps some of those in 32-bit and sums in other orders; it does not
    round more often)."""
    if dtype == "float32":
        return 3e-5
    rounded = reference(cfg, tensors, requests, rnd=bf16_rounding)
    return 2.0 * max(float((rounded[r] - exact[r]).abs().max()) / float(exact[r].abs().max()) for r in requests)


def check_rows(rows, exact, requests, allowed: float, what: str = "") -> float:
    worst = 0.0
    for rid, toks in requests.items():
        ref = exact[rid]
        scale = float(ref.abs().max())
        assert sorted(rows[rid]) == list(range(len(toks))), f"{what} request {rid}: not every position came back"
        got = torch.stack([rows[rid][p] for p in range(len(toks))]).double()
        assert torch.isfinite(got).all(), f"{what} request {rid}: logits that are not numbers"
        err = (got - ref).abs().max(dim=1).values / scale
        bad = (err > allowed).nonzero()
        assert len(bad) == 0, (f"{what} request {rid}: first wrong position {int(bad[0])} of {len(toks)} (error "
                               f"{float(err[int(bad[0])]):.3e} of the largest logit, allowed {allowed:.1e}); {len(bad)} positions wrong")
        worst = max(worst, float(err.max()))
    return worst

"""Small Gokosun configurations for the tests, their random weights, and the comparison with the plain decoder.

The configurations differ from one another in every size and option: matrix memories with key channels narrower and
wider than their values and caps small and large, latent attention with query and key vectors narrower and wider than
the heads they feed and rotated parts of two to thirty-two features with and without bent frequencies, grouped-query
attention with one, several or all query heads to a key head, values of another width than keys, rotations over none,
part or all of a head, layers that mix their values with the first such layer's and layers that do not, dense and
routed feed-forwards with and without a shared expert, layers without a feed-forward, sizes that are multiples of
nothing.
"""
from __future__ import annotations

import os
from typing import Dict, List

import torch

from llm_rs_amd import GokosunConfig, random_model_tensors, write_model_folder
from plain_gokosun import bf16_rounding, plain_gokosun_logits


def dense(ff, limit=1.0):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff, limit=1.5, scale=2.0, shared=None):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "scale": scale},
            "shared": None if shared is None else {"ff": shared[0], "limit": shared[1]}}


def mlstm(heads, dim, vdim, cap=15.0, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base=10000.0, scaling=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
         "rot": {"dims": rot_dim, "base": base, "scaling": scaling}}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def attention(heads, kv_heads, dim, vdim, scale, rot_dims=None, base=10000.0, v_mix=False, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix,
         "rot": None if rot_dims is None else {"dims": rot_dims, "base": base}}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def config(width, vocab, layers, eps=1e-5):
    return {"architecture": "Gokosun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


BENT = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 2.0}

ODD = config(46, 97, [
    attention(6, 2, 10, 6, 0.3, rot_dims=6, base=100.0, v_mix=True, mlp=moe(5, 2, 7, limit=0.7, scale=1.5, shared=(9, 2.5))),
    mlstm(3, 5, 7, cap=4.0, mlp=dense(30, 0.8)),
    latent(3, 5, 2, 7, 9, 11, 0.4, base=50.0, scaling=BENT, mlp=dense(11, 3.0)),
    attention(3, 1, 12, 20, 0.7, rot_dims=12),
    attention(2, 2, 8, 6, 0.5, rot_dims=None, v_mix=True, mlp=moe(3, 3, 5, shared=None)),
    mlstm(1, 13, 4, cap=30.0, mlp=moe(4, 1, 6, scale=0.5, shared=(3, 1.0))),
])
PLAIN = config(64, 128, [
    latent(4, 16, 8, 16, 24, 40, 0.2, mlp=dense(96)),
    mlstm(2, 16, 32, mlp=dense(48, 2.0)),
    attention(4, 1, 16, 16, 0.25, rot_dims=8, v_mix=True, mlp=moe(4, 2, 32, shared=(16, 2.0))),
    attention(2, 1, 32, 16, 0.2, rot_dims=32, v_mix=True, mlp=dense(64)),
], eps=1e-6)
# widths at which the bfloat16 products go to the matrix cores, heads and latent widths the matrix-core attention takes
WIDE = config(320, 352, [
    attention(8, 2, 64, 64, 0.125, rot_dims=32, base=500.0, v_mix=True, mlp=moe(6, 2, 128, shared=(64, 2.0))),
    latent(8, 32, 32, 32, 96, 128, 0.2, scaling=BENT, mlp=dense(512)),
    mlstm(4, 64, 64, mlp=dense(256, 1.5)),
    latent(16, 64, 64, 32, 192, 64, 0.1),
    mlstm(2, 128, 96, cap=8.0, mlp=moe(8, 3, 64)),
    attention(4, 4, 32, 96, 0.2, rot_dims=32, v_mix=False, mlp=dense(128)),
    attention(4, 2, 64, 64, 0.15, rot_dims=64, v_mix=True),
])
CONFIGS = {"odd": ODD, "plain": PLAIN, "wide": WIDE}
PAGE_SIZE = {"odd": 4, "plain": 16, "wide": 16}


def one_layer(layer, width=40, vocab=61, eps=1e-5):
    return config(width, vocab, [layer], eps)


def loud(tensors) -> None:
    """Random weights under which what a mixer does shows: queries enlarged so that scores spread, the mixers' outputs
    enlarged so that they count beside the stream, and routers enlarged so that the choice of experts is no near tie."""
    for name in list(tensors):
        factor = (4.0 if name.endswith((".mix.q", ".mix.uq")) else 4.0 if name.endswith(".mix.o") else 2.0 if name.endswith(".mlp.router")
                  else 3.0 if name.endswith(".mlp.correction") else None)
        if factor is not None:
            tensors[name] = (tensors[name].double() * factor).to(tensors[name].dtype)


def calm_routers(tensors) -> None:
    """Routers under which 16-bit rounding of their input cannot change which experts a token gets (two choice scores
    that differ by less than the rounding would otherwise fall either way, and an expert swapped for another is no
    rounding error): the logits hardly move with the token, and the corrections lie 0.05 apart.  The weights still
    differ from token to token.  Which experts a token gets by its own scores is what the 32-bit runs check."""
    for name in list(tensors):
        if name.endswith(".mlp.router"):
            tensors[name] = (tensors[name].double() * 0.025).to(tensors[name].dtype)
        elif name.endswith(".mlp.correction"):
            n = tensors[name].numel()
            order = torch.tensor([(5 * e + 2) % n if n % 5 else (3 * e + 1) % n for e in range(n)], dtype=torch.float64)
            assert len(set(order.tolist())) == n
            tensors[name] = (0.05 * order).to(tensors[name].dtype)


def make_model(cfg: dict, seed: int = 0, change=None, calm_router: bool = False):
    """(typed config, {name: bfloat16 tensor}); `change(tensors)` may put values of its own in."""
    typed = GokosunConfig.from_dict(cfg)
    tensors = random_model_tensors(typed, seed)
    loud(tensors)
    if calm_router:
        calm_routers(tensors)
    if change is not None:
        change(tensors)
    return typed, tensors


def make_folder(tmp_path, cfg: dict, seed: int = 0, change=None, name: str = "model", calm_router: bool = False) -> str:
    typed, tensors = make_model(cfg, seed, change, calm_router)
    folder = os.path.join(str(tmp_path), name)
    write_model_folder(folder, typed, tensors)
    return folder


def reference(cfg: dict, tensors, requests: Dict[str, List[int]], rnd=None):
    kw = {} if rnd is None else {"rnd": rnd}
    return {rid: plain_gokosun_logits(cfg, tensors, toks, **kw) for rid, toks in requests.items()}


def allowed_error(dtype: str, cfg: dict, tensors, requests, exact) -> float:
    """How far the engine may be from the exact logits, as a part of a sequence's largest logit.  float32: 3e-5.
    bfloat16: twice as far as the plain decoder gets when every activation that passes through memory between two
    stages is rounded to bfloat16 (the engine keeps some of those in 32-bit and sums in other orders; it does not
    round more often)."""
    if dtype == "float32":
        return 3e-5
    rounded = reference(cfg, tensors, requests, rnd=bf16_rounding)
    return 2.0 * max(float((rounded[r] - exact[r]).abs().max()) / float(exact[r].abs().max()) for r in requests)


def check_rows(rows, exact, requests, allowed: float, what: str = "", few_may_pass: bool = False) -> float:
    """Every position of every request within `allowed` of the exact logits.  few_may_pass (for bfloat16 only): one
    position in fifty of a request (at least one) may be up to 1.5 times as far.  A matrix memory divides its read-out
    by |n . q|, which passes close to its floor now and then, and what was rounded before is enlarged there beyond any
    bound that the other positions' errors give."""
    worst = 0.0
    for rid, toks in requests.items():
        ref = exact[rid]
        scale = float(ref.abs().max())
        assert sorted(rows[rid]) == list(range(len(toks))), f"{what} request {rid}: not every position came back"
        got = torch.stack([rows[rid][p] for p in range(len(toks))]).double()
        assert torch.isfinite(got).all(), f"{what} request {rid}: logits that are not numbers"
        err = (got - ref).abs().max(dim=1).values / scale
        bad = (err > allowed).nonzero()
        if few_may_pass and 0 < len(bad) <= max(1, len(toks) // 50) and float(err.max()) <= 1.5 * allowed:
            bad = bad[:0]
        assert len(bad) == 0, (f"{what} request {rid}: first wrong position {int(bad[0])} of {len(toks)} (error "
                               f"{float(err[int(bad[0])]):.3e} of the largest logit, allowed {allowed:.1e}); {len(bad)} positions wrong")
        worst = max(worst, float(err.max()))
    return worst

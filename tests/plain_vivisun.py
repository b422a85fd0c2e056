"""A plain, slow Vivisun decoder for the tests to compare the engine with.

Whole sequences, no cache, no batching, one function per mechanism, in ordinary
tensor operations and explicit loops.  It shares no code with the package.
Computation is in `compute` (float64 by default) from the weights as stored.

The design: a token table; layers whose two halves read the same stream,
x <- x + mixer(norm1(x)) + ff(norm2(x)); every norm a dynamic tanh,
tanh(alpha x) w + b; a mixer that is either softmax attention (short causal
convolutions on q, k and v, an RMS norm of q and k per head, a rotation of part
of each head in the half-split layout with frequencies bent by wavelength and
an enlarged cosine and sine, a sigmoid gate on the heads' outputs) or latent
attention (keys and values of all heads expanded from one small normed vector
per token, no positions, a learned sink in the softmax's denominator, a
sigmoid gate per head); a gated feed-forward with silu; a stretch of layers
that runs several times with the same weights, the token embeddings added to
the stream again before every pass but the first; a final norm and an output
matrix.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional, Sequence

import torch

# `rnd`: applied to every activation that one stage hands the next through memory in an implementation that keeps
# such hand-overs in 16 bits (never to the stream, a score, a softmax weight or a norm's sum).  The identity by default.
_same = lambda x: x


def bf16_rounding(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


def plain_rmsnorm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def plain_sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def plain_silu(x):
    return x * plain_sigmoid(x)


def plain_dyt(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, alpha: torch.Tensor) -> torch.Tensor:
    """Dynamic tanh: no mean, no variance; one scalar in front of the tanh, a weight and a bias per feature behind it."""
    return torch.tanh(alpha * x) * w + b


def plain_causal_conv(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """u: [T, C]; taps: [C, n].  y_t = sum_j taps[:, j] u_(t - n + 1 + j): the last tap is the current token's, and what
    lies before the sequence is zero."""
    T, C = u.shape
    n = taps.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(n):
            s = t - n + 1 + j
            if s >= 0:
                y[t] += taps[:, j] * u[s]
    return y


def plain_bent_frequencies(rot: dict) -> (torch.Tensor, float):
    """f_i = base^(-2i/dims) for i < dims/2, bent between two wavelengths: with
    d(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), dims - 1),
    r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the frequency is f_i / factor r_i + f_i (1 - r_i); cosine and sine
    are both multiplied by 0.1 ln(factor) + 1.  Returns (frequencies in float64, that multiplier)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc is None:
        return torch.tensor(f, dtype=torch.float64), 1.0
    factor, original = float(sc["factor"]), float(sc["original"])
    d = lambda t: dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo = max(math.floor(d(float(sc["fast"]))), 0)
    hi = min(math.ceil(d(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * r + fi * (1.0 - r))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(factor) + 1.0


def plain_rotate_half(x: torch.Tensor, positions: Sequence[int], freq: torch.Tensor, gain: float) -> torch.Tensor:
    """x: [T, heads, dim]; the first 2 * len(freq) features of each head are rotated, feature i together with feature
    i + len(freq): (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * freq_i, cosine and sine times gain."""
    n = freq.shape[0]
    if n == 0:
        return x
    ang = torch.tensor(list(positions), dtype=torch.float64)[:, None] * freq[None, :]
    cos, sin = (torch.cos(ang) * gain).to(x.dtype)[:, None, :], (torch.sin(ang) * gain).to(x.dtype)[:, None, :]
    u, v = x[..., :n], x[..., n:2 * n]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., 2 * n:]], dim=-1)


def plain_softmax_rows(scores: torch.Tensor, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """scores: [heads, T, T] with -inf where a key is hidden; sink: [heads] or None.  With a sink the denominator also
    holds exp(sink_h), once, for every query: a key without a value."""
    m = scores.max(dim=-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None, None])
    e = torch.exp(scores - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink[:, None, None] - m)
    return e / den


def plain_causal_mask(T: int, dtype) -> torch.Tensor:
    i = torch.arange(T)
    return torch.where(i[None, :] <= i[:, None], 0.0, float("-inf")).to(dtype)


def plain_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, rnd: Callable = _same) -> torch.Tensor:
    """h: [T, D], the mixer's input."""
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"]), int(m["vdim"])
    q, k, v = h @ w["q"].T, h @ w["k"].T, h @ w["v"].T
    if int(m.get("conv") or 0) > 0:
        q, k, v = plain_causal_conv(q, w["q.conv"]), plain_causal_conv(k, w["k.conv"]), plain_causal_conv(v, w["v.conv"])
    q = plain_rmsnorm(q.view(T, H, dk), w["q.norm"], eps)
    k = plain_rmsnorm(k.view(T, G, dk), w["k.norm"], eps)
    v = rnd(v).view(T, G, dv)
    rot = m.get("rot")
    if rot is not None and int(rot["dims"]) > 0:
        freq, gain = plain_bent_frequencies(rot)
        q, k = plain_rotate_half(q, range(T), freq, gain), plain_rotate_half(k, range(T), freq, gain)
    q, k = rnd(q), rnd(k)
    per = H // G
    kk, vv = k.repeat_interleave(per, dim=1), v.repeat_interleave(per, dim=1)      # query head a uses key head a // per
    scores = torch.einsum("ihd,jhd->hij", q, kk) * float(m["scale"]) + plain_causal_mask(T, h.dtype)[None]
    p = plain_softmax_rows(scores)
    o = rnd(torch.einsum("hij,jhd->ihd", p, vv)).reshape(T, H * dv)
    o = o * plain_sigmoid(h @ w["g"].T)
    return rnd(o) @ w["o"].T


def plain_latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, rnd: Callable = _same) -> torch.Tensor:
    """h: [T, D].  One normed vector c of kv_rank numbers per token; every head's keys and values are matrices times c."""
    T = h.shape[0]
    H, dk, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = rnd(h @ w["q"].T).view(T, H, dk)
    c = rnd(plain_rmsnorm(h @ w["dkv"].T, w["dkv.norm"], eps))
    k = rnd(c @ w["uk"].T).view(T, H, dk)
    v = rnd(c @ w["uv"].T).view(T, H, dv)
    scores = torch.einsum("ihd,jhd->hij", q, k) * float(m["scale"]) + plain_causal_mask(T, h.dtype)[None]
    p = plain_softmax_rows(scores, w["sink"])
    o = rnd(torch.einsum("hij,jhd->ihd", p, v))                    # [T, H, dv]
    o = o * plain_sigmoid(h @ w["g"].T)[:, :, None]                # one gate per head
    return rnd(o.reshape(T, H * dv)) @ w["o"].T


def plain_gated_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], rnd: Callable = _same) -> torch.Tensor:
    return rnd(plain_silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


MIXERS = {"attention": plain_attention, "latent_attention": plain_latent_attention}


def plain_schedule(n_layers: int, loop: Optional[dict]) -> List[tuple]:
    """(layer, whether the embeddings are added again right before it) in the order the layers run."""
    if not loop or int(loop.get("times", 1)) <= 1 or int(loop["stop"]) <= int(loop["start"]):
        return [(i, False) for i in range(n_layers)]
    a, b, n = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(a)]
    for p in range(n):
        order += [(i, p > 0 and i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n_layers)]


def _under(tensors: Dict[str, torch.Tensor], prefix: str, compute) -> Dict[str, torch.Tensor]:
    return {n[len(prefix):]: t.to(compute) for n, t in tensors.items() if n.startswith(prefix)}


def plain_vivisun_logits(config: dict, tensors: Dict[str, torch.Tensor], tokens: Sequence[int], compute=torch.float64,
                         rnd: Callable = _same, after_run: Optional[Callable] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence.  `after_run(run, x)` sees the stream after every layer run."""
    eps = float(config["norm"]["eps"])
    t = lambda n: tensors[n].to(compute)
    dyt = lambda x, name: plain_dyt(x, t(name), t(name + ".b"), t(name + ".alpha"))
    x0 = t("embed")[torch.as_tensor(list(tokens), dtype=torch.long)]
    x = x0.clone()
    for run, (i, again) in enumerate(plain_schedule(len(config["layers"]), config.get("loop"))):
        layer = config["layers"][i]
        if again:
            x = x + x0
        y = MIXERS[layer["type"]](rnd(dyt(x, f"l{i}.norm1")), _under(tensors, f"l{i}.mix.", compute), layer["mixer"], eps, rnd)
        if layer.get("mlp") is not None:
            y = y + plain_gated_ff(rnd(dyt(x, f"l{i}.norm2")), _under(tensors, f"l{i}.mlp.", compute), rnd)
        x = x + y
        if after_run is not None:
            after_run(run, x)
    return rnd(dyt(x, "final.norm")) @ t("head").T

"""A plain, slow Gokosun decoder for the tests to compare the engine with.

Whole sequences, no cache, no batching, one function per mechanism, in ordinary
tensor operations and explicit loops.  It shares no code with the package.
Computation is in `compute` (float64 by default) from the weights as stored.

The design: a token table; layers with one layer norm (weight and bias) whose
output both halves read, x <- x + (mixer(n) + ff(n)) with n = norm1(x); a mixer
that is a matrix memory with exponential gates (mLSTM: per head a matrix S and a
vector n that decay by a forget gate and take k v^T and k under an input gate,
kept in range by a running maximum of the gates' logarithms), latent attention
(queries through a small normed vector, keys and values of all heads expanded
from another, one rotated key part shared by the heads, frequencies bent between
two wavelengths, a learned sink in the softmax's denominator) or grouped-query
attention (q and k RMS-normed over the whole projection, part of each head
rotated in the half-split layout, the values of later layers mixed with the first
such layer's); a feed-forward with a clamped, gated activation, dense or as a
mixture of experts chosen by sigmoid scores plus a correction, beside a shared
expert; a final layer norm and an output matrix.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional, Sequence

import torch

# `rnd`: applied to every activation that one stage hands the next through memory in an implementation that keeps
# such hand-overs in 16 bits (never to the stream, a score, a softmax weight, a norm's sum, a gate of the recurrence or
# its state).  The identity by default.
_same = lambda x: x


def bf16_rounding(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


def plain_sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def plain_layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * w + b


def plain_rmsnorm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def plain_frequencies(rot: dict) -> (torch.Tensor, float):
    """The rotation's frequencies, one for each pair, and what cosine and sine are multiplied by."""
    dims, base = int(rot["dims"]), float(rot["base"])
    freq = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    gain = 1.0
    sc = rot.get("scaling")
    if sc is not None:
        factor, original = float(sc["factor"]), float(sc["original"])
        where = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(where(float(sc["fast"]))), 0)
        hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
        for i in range(dims // 2):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            freq[i] = freq[i] / factor * ramp + freq[i] * (1.0 - ramp)
        gain = 0.1 * math.log(factor) + 1.0
    return torch.tensor(freq, dtype=torch.float64), gain


def plain_rotate(x: torch.Tensor, positions: Sequence[int], freq: torch.Tensor, gain: float, layout: str) -> torch.Tensor:
    """x: [T, heads, d].  The first 2 len(freq) features of every head are turned; pair i is (i, i + len(freq)) in the
    layout "half" and (2i, 2i + 1) in "pairs"."""
    n = freq.numel()
    out = x.clone()
    for t, p in enumerate(positions):
        for i in range(n):
            a = float(p) * float(freq[i])
            c, s = math.cos(a) * gain, math.sin(a) * gain
            i0, i1 = (i, i + n) if layout == "half" else (2 * i, 2 * i + 1)
            u, v = x[t, :, i0], x[t, :, i1]
            out[t, :, i0] = u * c - v * s
            out[t, :, i1] = v * c + u * s
    return out


def plain_softmax_rows(scores: torch.Tensor, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """scores: [heads, T, T] with -inf where a key is not seen; sink: [heads] or None.  The sink joins the denominator
    once: it has no key and no value."""
    top = scores.max(dim=-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink.view(-1, 1, 1))
    e = torch.exp(scores - top)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink.view(-1, 1, 1) - top)
    return e / den


def plain_causal_mask(T: int, dtype) -> torch.Tensor:
    m = torch.zeros(T, T, dtype=dtype)
    m[torch.triu(torch.ones(T, T, dtype=torch.bool), diagonal=1)] = float("-inf")
    return m


def plain_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, v_first: Optional[torch.Tensor],
                    rnd: Callable = _same):
    """Grouped-query attention.  Returns (output [T, width], the values that were cached [T, kv_heads, vdim]).
    v_first: the first value-mixing layer's values, or None (this is that layer, or the layer mixes nothing)."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = plain_rmsnorm(h @ w["q"].T, w["q.norm"], eps).view(T, H, d)
    k = plain_rmsnorm(h @ w["k"].T, w["k.norm"], eps).view(T, G, d)
    v = (h @ w["v"].T).view(T, G, dv)
    rot = m.get("rot")
    if rot is not None and int(rot["dims"]) > 0:
        freq, gain = plain_frequencies(rot)
        q = plain_rotate(q, range(T), freq, gain, "half")
        k = plain_rotate(k, range(T), freq, gain, "half")
    if m.get("v_mix") and v_first is not None:
        lam = w["vmix"]
        v = (1.0 - lam) * v + lam * v_first
    q, k, v = rnd(q), rnd(k), rnd(v)
    mask = plain_causal_mask(T, h.dtype)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head, :] @ k[:, g, :].T) * float(m["scale"]) + mask
        p = plain_softmax_rows(s.unsqueeze(0))[0]
        out[:, head, :] = rnd(p) @ v[:, g, :]
    return rnd(out.reshape(T, H * dv)) @ w["o"].T, v


def plain_latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, rnd: Callable = _same) -> torch.Tensor:
    T = h.shape[0]
    H, d, r, dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    cq = rnd(plain_rmsnorm(h @ w["dq"].T, w["dq.norm"], eps))
    q = (cq @ w["uq"].T).view(T, H, d + r)
    q_flat, q_rot = q[:, :, :d], q[:, :, d:]
    low = h @ w["dkv"].T
    c = rnd(plain_rmsnorm(low[:, :rank], w["dkv.norm"], eps))
    k_rot = low[:, rank:].view(T, 1, r)
    freq, gain = plain_frequencies(m["rot"])
    q_rot = rnd(plain_rotate(q_rot, range(T), freq, gain, "pairs"))
    k_rot = rnd(plain_rotate(k_rot, range(T), freq, gain, "pairs"))[:, 0, :]
    q_flat = rnd(q_flat)
    k_flat = rnd((c @ w["uk"].T).view(T, H, d))
    v = rnd((c @ w["uv"].T).view(T, H, dv))
    mask = plain_causal_mask(T, h.dtype)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        s = (q_flat[:, head, :] @ k_flat[:, head, :].T + q_rot[:, head, :] @ k_rot.T) * float(m["scale"]) + mask
        p = plain_softmax_rows(s.unsqueeze(0), w["sink"][head:head + 1])[0]
        out[:, head, :] = rnd(p) @ v[:, head, :]
    return rnd(out.reshape(T, H * dv)) @ w["o"].T


def plain_mlstm_gates(h: torch.Tensor, w: Dict[str, torch.Tensor], cap: float):
    """The logarithms of the input and the forget gate, [T, heads] each."""
    i = cap * torch.tanh((h @ w["i"].T + w["i.b"]) / cap)
    z = cap * torch.tanh((h @ w["f"].T + w["f.b"]) / cap)
    f = -torch.log1p(torch.exp(-z))           # log sigmoid
    return i, f


def plain_mlstm_head(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, i: torch.Tensor, f: torch.Tensor, state=None):
    """One head, token by token.  q, k: [T, d] (q already scaled); v: [T, dv]; i, f: [T].  state: (S [d, dv], n [d], m) or
    None for the start, where all three are zero.  Returns (read-outs [T, dv], the state after the last token)."""
    T, d = q.shape
    dv = v.shape[1]
    if state is None:
        S, n, m = torch.zeros(d, dv, dtype=q.dtype), torch.zeros(d, dtype=q.dtype), torch.zeros((), dtype=q.dtype)
    else:
        S, n, m = state
    out = torch.zeros(T, dv, dtype=q.dtype)
    for t in range(T):
        m_new = torch.maximum(f[t] + m, i[t])
        keep, take = torch.exp(f[t] + m - m_new), torch.exp(i[t] - m_new)
        S = keep * S + take * torch.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_new
        den = torch.maximum(torch.abs(n @ q[t]), torch.exp(-m)) + 1e-6
        out[t] = (S.T @ q[t]) / den
    return out, (S, n, m)


def plain_mlstm(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, rnd: Callable = _same) -> torch.Tensor:
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w["q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w["k"].T).view(T, H, d)
    v = (h @ w["v"].T).view(T, H, dv)
    i, f = plain_mlstm_gates(h, w, float(m["gate_cap"]))
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        o, _ = plain_mlstm_head(q[:, head], k[:, head], v[:, head], i[:, head], f[:, head])
        out[:, head] = plain_rmsnorm(o, None, eps)
    y = out.reshape(T, H * dv) * w["norm"] * plain_sigmoid(h @ w["g"].T)
    return rnd(y) @ w["o"].T


def plain_clamped_glu(h: torch.Tensor, w: Dict[str, torch.Tensor], limit: float, rnd: Callable = _same) -> torch.Tensor:
    g = torch.clamp(h @ w["gate"].T, max=limit)
    u = torch.clamp(h @ w["up"].T, min=-limit, max=limit)
    return rnd(g * plain_sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def plain_route(h: torch.Tensor, w: Dict[str, torch.Tensor], top: int, scale: float):
    """(chosen experts [T, top], their weights [T, top])."""
    s = plain_sigmoid(h @ w["router"].T)
    chosen = torch.topk(s + w["correction"], top, dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(dim=-1, keepdim=True) + 1e-20) * scale


def _under(tensors: Dict[str, torch.Tensor], prefix: str, compute=None) -> Dict[str, torch.Tensor]:
    return {n[len(prefix):]: (t if compute is None else t.to(compute)) for n, t in tensors.items() if n.startswith(prefix)}


def plain_experts(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict, rnd: Callable = _same) -> torch.Tensor:
    top, scale = int(mlp["router"]["top"]), float(mlp["router"]["scale"])
    chosen, weights = plain_route(h, w, top, scale)
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(chosen[t, j])
            out[t] += weights[t, j] * plain_clamped_glu(h[t:t + 1], _under(w, f"e{e}."), float(mlp["expert"]["limit"]), rnd)[0]
    if mlp.get("shared") is not None:
        out = out + plain_clamped_glu(h, _under(w, "shared."), float(mlp["shared"]["limit"]), rnd)
    return out


def plain_feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict, rnd: Callable = _same) -> torch.Tensor:
    if mlp.get("kind", "dense") == "dense":
        return plain_clamped_glu(h, w, float(mlp["limit"]), rnd)
    return plain_experts(h, w, mlp, rnd)


def plain_gokosun_logits(config: dict, tensors: Dict[str, torch.Tensor], tokens: Sequence[int], compute=torch.float64,
                         rnd: Callable = _same, after_layer: Optional[Callable] = None) -> torch.Tensor:
    """Logits [T, vocab] of the whole sequence.  `after_layer(i, x)` sees the stream after every layer."""
    eps = float(config["norm"]["eps"])
    x = tensors["embed"].to(compute)[torch.tensor(list(tokens), dtype=torch.long)]
    v_first = None
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        n = rnd(plain_layernorm(x, tensors[p + "norm1"].to(compute), tensors[p + "norm1.b"].to(compute), eps))
        w = _under(tensors, p + "mix.", compute)
        kind, m = layer["type"], layer["mixer"]
        if kind == "mlstm":
            y = plain_mlstm(n, w, m, eps, rnd)
        elif kind == "latent_attention":
            y = plain_latent_attention(n, w, m, eps, rnd)
        elif kind == "attention":
            y, v = plain_attention(n, w, m, eps, v_first, rnd)
            if m.get("v_mix") and v_first is None:
                v_first = v
        else:
            raise ValueError(f"unknown mixer {kind!r}")
        if layer.get("mlp") is not None:
            y = y + plain_feed_forward(n, _under(tensors, p + "mlp.", compute), layer["mlp"], rnd)
        x = x + y
        if after_layer is not None:
            after_layer(i, x)
    n = rnd(plain_layernorm(x, tensors["final.norm"].to(compute), tensors["final.norm.b"].to(compute), eps))
    return n @ tensors["head"].to(compute).T

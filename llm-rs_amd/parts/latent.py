"""Latent attention(hidden_size, heads, dim, vdim, kv_rank, scale, eps, sink, gate): causal softmax attention whose keys
and values are all made from one small vector per token.

  q = Wq x [heads, dim];  c = rmsnorm(Wdkv x) * dkv.norm [kv_rank];  k_h = Wuk_h c,  v_h = Wuv_h c
  s_ij = (q_hi . k_hj) * scale, causal, no positions;  softmax over the visible keys, with `sink` the denominator also
  holds exp(sink_h) once (a key without a value);  o_h = sum_j p_ij v_hj, times sigmoid(Wg x)_h (`gate` = "head"),
  through Wo.

Only c is cached, and keys and values are never expanded: q_h . (Wuk_h c_j) = (Wuk_h^T q_h) . c_j, and
sum_j p_ij Wuv_h c_j = Wuv_h (sum_j p_ij c_j).  So a step is: one product for q | dkv | gate (32-bit sums); c normed and
written into its pages, once as rows (for the scores) and once transposed (for the weighted sum, cache_layout.h: the
paged cache of one key head of width kv_rank whose values are its keys); every head's query carried into the latent
space by its own small matrix (`head_product`); attention of `heads` query heads over the one latent head, with the
sink; every head's result carried out of the latent space by its own small matrix, the gate applied to the 32-bit sums
on the way; the output projection adds into the stream.  Scores, softmax, sink, norm and gate are 32-bit.

Two further parameters, for designs that have them:
  q_rank: the queries pass a latent vector of their own, c_q = rmsnorm(Wdq x) * dq.norm [q_rank], q = Wuq c_q;
  rot_dim (with `position`, a rotation in neighbouring pairs): every head's query has rot_dim more features behind its
    dim, and Wdkv x has rot_dim more rows behind the latent vector, one key part shared by all heads; both are rotated
    by position, and the score is (q_h . k_h + q_rot_h . k_rot) * scale.  The rotated key part is cached behind c, so the
    latent head is kv_rank + rot_dim wide; a head's query there is [Wuk_h^T q_h, q_rot_h] (its small matrix passes the
    rotated features through), and the matrix that carries results out has zeros for the rotated part's columns.
"""
from __future__ import annotations

import torch

from ..cache.spec import PagedKV
from ..kernels import EPI_ACCUM_F32, EPI_STORE_F32, kernels
from .attention import KeyedBySplitChunk
from .base import Mixer, TensorSpec, build_position, place, register_mixer


class LatentAttention(KeyedBySplitChunk, Mixer):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.heads = int(p["hidden_size"]), int(p["heads"])
        self.dk, self.dv, self.rank = int(p["dim"]), int(p["vdim"]), int(p["kv_rank"])
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.has_sink = bool(p.get("sink", False))
        self.gate = p.get("gate")
        if self.gate not in (None, "head"):
            raise ValueError(f"unknown output gate {self.gate!r} (known: head)")
        self.q_rank, self.rot = int(p.get("q_rank") or 0), int(p.get("rot_dim") or 0)
        self.width = self.rank + self.rot           # of the latent head: c, then the rotated key part
        if self.width > 512:        # the attention kernels' widest head, which the latent vector is here
            raise ValueError(f"a latent vector of {self.rank} numbers with a rotated part of {self.rot} exceeds the 512 that the attention kernels take")
        self.position = build_position(p.get("position"), dtype) if self.rot > 0 else None
        if self.rot > 0:
            rotary = self.position.rotary() if self.position is not None else None
            if rotary is None or not rotary[2] or rotary[1] != self.rot:
                raise ValueError("the rotated part needs a rotation in neighbouring pairs over all its features")
        self.gain = float(getattr(self.position, "gain", 1.0)) if self.position is not None else 1.0
        self.recording_signature = ("attention", 1, self.width, 0)
        leaves = {"q": "q", "dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv",
                  "sink": "sink", "gate": "g", "o": "o", **(p.get("names") or {})}
        self.names = {key: self.name(leaf) for key, leaf in leaves.items()}
        self.qh = self.dk + self.rot                # a head's query features: dim, then the rotated ones
        self.q_size, self.o_size = self.heads * self.qh, self.heads * self.dv
        self.q_part = self.q_rank or self.q_size    # columns of the input product that belong to the queries
        self.n_gate = self.heads if self.gate else 0
        self.w_in = self.w_o = self.w_uk_t = self.w_uv = self.norm = self.sink = self.w_uq = self.q_norm = None

    def tensors(self):
        n, D = self.names, self.hidden
        t = {n["dkv"]: TensorSpec((self.width, D)), n["dkv_norm"]: TensorSpec((self.rank,), "norm"),
             n["uk"]: TensorSpec((self.heads * self.dk, self.rank), "normal:0.0:0.1"), n["uv"]: TensorSpec((self.o_size, self.rank), "normal:0.0:0.1"),
             n["o"]: TensorSpec((D, self.o_size))}
        if self.q_rank:
            t[n["dq"]] = TensorSpec((self.q_rank, D))
            t[n["dq_norm"]] = TensorSpec((self.q_rank,), "norm")
            t[n["uq"]] = TensorSpec((self.q_size, self.q_rank), "normal:0.0:0.1")
        else:
            t[n["q"]] = TensorSpec((self.q_size, D))
        if self.has_sink:
            t[n["sink"]] = TensorSpec((self.heads,), "normal:0.0:1.0")
        if self.gate:
            t[n["gate"]] = TensorSpec((self.heads, D))
        return t

    def _rotated_first(self, w: torch.Tensor, undo: bool = False) -> torch.Tensor:
        """Rows of a query weight reordered within each head, from [dim, rotated] to [rotated, dim] (the kernel that
        finishes q turns a head's first features); `undo` puts them back."""
        if self.rot == 0:
            return w
        order = torch.cat([torch.arange(self.dk, self.qh), torch.arange(self.dk)])
        if undo:
            order = torch.argsort(order)
        return w.view(self.heads, self.qh, -1)[:, order.to(w.device), :].reshape(w.shape).contiguous()

    def load(self, tensors, device):
        n = self.names
        get = lambda key: place(tensors[n[key]], device, self.dtype)
        H, R, r = self.heads, self.rank, self.rot
        if self.q_rank:
            first = get("dq")
            self.w_uq = self._rotated_first(get("uq"))
            self.q_norm = place(tensors[n["dq_norm"]], device, torch.float32)
        else:
            first = self._rotated_first(get("q"))
        self.w_in = torch.cat([first, get("dkv")] + ([get("gate")] if self.gate else []), dim=0).contiguous()
        # per head [out, in]: into the latent space by Wuk_h^T [kv_rank, dim], out of it by Wuv_h [vdim, kv_rank]; with a
        # rotated part a head's query is [rotated, dim] -> [Wuk_h^T q, rotated], and results have nothing of the part
        uk_t = get("uk").view(H, self.dk, R).transpose(1, 2)
        self.w_uk_t = torch.zeros(H, self.width, self.qh, dtype=self.dtype, device=uk_t.device)
        self.w_uk_t[:, :R, r:] = uk_t
        if r:
            self.w_uk_t[:, R:, :r] = torch.eye(r, dtype=self.dtype, device=uk_t.device)
        self.w_uv = torch.zeros(H, self.dv, self.width, dtype=self.dtype, device=uk_t.device)
        self.w_uv[:, :, :R] = get("uv").view(H, self.dv, R)
        self.w_o = get("o")
        if self.position is not None:
            self.position.to(device)
        self.norm = place(tensors[n["dkv_norm"]], device, torch.float32)
        self.sink = place(tensors[n["sink"]], device, torch.float32) if self.has_sink else None

    def export(self):
        n, w = self.names, self.w_in.cpu()
        Q, R, r = self.q_part, self.rank, self.rot
        out = {n["dkv"]: w[Q:Q + self.width].contiguous(), n["dkv_norm"]: self.norm.cpu(), n["o"]: self.w_o.cpu(),
               n["uk"]: self.w_uk_t.cpu()[:, :R, r:].transpose(1, 2).reshape(self.heads * self.dk, R).contiguous(),
               n["uv"]: self.w_uv.cpu()[:, :, :R].reshape(self.o_size, R).contiguous()}
        if self.q_rank:
            out[n["dq"]] = w[:Q].contiguous()
            out[n["dq_norm"]] = self.q_norm.cpu()
            out[n["uq"]] = self._rotated_first(self.w_uq.cpu(), undo=True)
        else:
            out[n["q"]] = self._rotated_first(w[:Q], undo=True)
        if self.has_sink:
            out[n["sink"]] = self.sink.cpu()
        if self.gate:
            out[n["gate"]] = w[Q + self.width:].contiguous()
        return out

    def cache_need(self):
        return PagedKV(1, self.width)          # one latent head; its keys are its values

    def forward(self, ctx, x, h, cache):
        k = kernels()
        T, H, R, Q = x.shape[0], self.heads, self.width, self.q_part
        g = cache.group
        sums = ctx.workspace("latent.sums", (T, self.w_in.shape[0]), torch.float32)
        k.gemm(x, self.w_in, sums, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_in))
        inv_freq = self.position.rotary()[0] if self.rot else None
        rotated = (self.rot, ctx.positions, inv_freq, self.gain) if self.rot else None
        first = ctx.workspace("latent.cq" if self.q_rank else "latent.q", (T, Q), self.dtype)
        k.latent_finish(sums, first, Q, self.rank, self.norm, self.eps, ctx.slot_maps[g], cache.k, cache.v, cache.page_size,
                        cache.num_pages, cache.writes, q_weight=self.q_norm, rotated=rotated)
        q = first
        if self.q_rank or self.rot:     # queries through their latent vector, and a head's first features turned
            q = ctx.workspace("latent.q", (T, self.q_size), self.dtype)
            if self.q_rank:
                qs = ctx.workspace("latent.qsums", (T, self.q_size), torch.float32)
                k.gemm(first, self.w_uq, qs, EPI_STORE_F32, ctx.gemm_workspace(first, self.w_uq))
            else:
                qs = sums[:, :Q]
            k.qkv_finish(qs, None, q, None, None, None, H, 0, self.qh, self.qh, cache.page_size, cache.num_pages, False, 0.0,
                         ctx.positions, inv_freq, self.rot, gain=self.gain)
        ql = ctx.workspace("latent.ql", (T, H * R), self.dtype)
        k.head_product(q, self.w_uk_t, ql)
        ol = ctx.workspace("latent.ol", (T, H * R), self.dtype)
        need = k.attention_scratch_floats(ctx.n_entries, H, R, ctx.max_seq_len, 1, ctx.n_single) if ctx.n_single else 0
        scratch = ctx.workspace("attn.partial", (need,), torch.float32) if need else None
        k.attention(ql, ol, cache.k, cache.v, ctx.block_tables[g], ctx.token_entry, ctx.positions, ctx.q_starts, ctx.seq_lens,
                    H, 1, R, cache.page_size, cache.num_pages, 0, self.scale, scratch, ctx.max_seq_len, ctx.n_single,
                    self._keys_for_the_split(ctx), sink=self.sink)
        o = ctx.workspace("latent.o", (T, self.o_size), self.dtype)
        k.head_product(ol, self.w_uv, o, gate=sums[:, Q + R:] if self.gate else None)
        k.gemm(o, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(o, self.w_o))
        ctx.note_left(h, None)


register_mixer("latent_attention", LatentAttention)

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
"""
from __future__ import annotations

import torch

from ..cache.spec import PagedKV
from ..kernels import EPI_ACCUM_F32, EPI_STORE_F32, kernels
from .attention import KeyedBySplitChunk
from .base import Mixer, TensorSpec, place, register_mixer


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
        if self.rank > 512:         # the attention kernels' widest head, which the latent vector is here
            raise ValueError(f"a latent vector of {self.rank} numbers exceeds the 512 that the attention kernels take")
        self.recording_signature = ("attention", 1, self.rank, 0)
        leaves = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "sink": "sink", "gate": "g", "o": "o",
                  **(p.get("names") or {})}
        self.names = {key: self.name(leaf) for key, leaf in leaves.items()}
        self.q_size, self.o_size = self.heads * self.dk, self.heads * self.dv
        self.n_gate = self.heads if self.gate else 0
        self.w_in = self.w_o = self.w_uk_t = self.w_uv = self.norm = self.sink = None

    def tensors(self):
        n, D = self.names, self.hidden
        t = {n["q"]: TensorSpec((self.q_size, D)), n["dkv"]: TensorSpec((self.rank, D)), n["dkv_norm"]: TensorSpec((self.rank,), "norm"),
             n["uk"]: TensorSpec((self.q_size, self.rank), "normal:0.0:0.1"), n["uv"]: TensorSpec((self.o_size, self.rank), "normal:0.0:0.1"),
             n["o"]: TensorSpec((D, self.o_size))}
        if self.has_sink:
            t[n["sink"]] = TensorSpec((self.heads,), "normal:0.0:1.0")
        if self.gate:
            t[n["gate"]] = TensorSpec((self.heads, D))
        return t

    def load(self, tensors, device):
        n = self.names
        get = lambda key: place(tensors[n[key]], device, self.dtype)
        self.w_in = torch.cat([get("q"), get("dkv")] + ([get("gate")] if self.gate else []), dim=0).contiguous()
        # per head [out, in]: into the latent space by Wuk_h^T [kv_rank, dim], out of it by Wuv_h [vdim, kv_rank]
        self.w_uk_t = get("uk").view(self.heads, self.dk, self.rank).transpose(1, 2).contiguous()
        self.w_uv = get("uv").view(self.heads, self.dv, self.rank).contiguous()
        self.w_o = get("o")
        self.norm = place(tensors[n["dkv_norm"]], device, torch.float32)
        self.sink = place(tensors[n["sink"]], device, torch.float32) if self.has_sink else None

    def export(self):
        n, w = self.names, self.w_in.cpu()
        out = {n["q"]: w[:self.q_size].contiguous(), n["dkv"]: w[self.q_size:self.q_size + self.rank].contiguous(),
               n["dkv_norm"]: self.norm.cpu(), n["o"]: self.w_o.cpu(),
               n["uk"]: self.w_uk_t.cpu().transpose(1, 2).reshape(self.q_size, self.rank).contiguous(),
               n["uv"]: self.w_uv.cpu().reshape(self.o_size, self.rank).contiguous()}
        if self.has_sink:
            out[n["sink"]] = self.sink.cpu()
        if self.gate:
            out[n["gate"]] = w[self.q_size + self.rank:].contiguous()
        return out

    def cache_need(self):
        return PagedKV(1, self.rank)           # one latent head; its keys are its values

    def forward(self, ctx, x, h, cache):
        k = kernels()
        T, H, R = x.shape[0], self.heads, self.rank
        g = cache.group
        sums = ctx.workspace("latent.sums", (T, self.w_in.shape[0]), torch.float32)
        k.gemm(x, self.w_in, sums, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_in))
        q = ctx.workspace("latent.q", (T, self.q_size), self.dtype)
        k.latent_finish(sums, q, self.q_size, R, self.norm, self.eps, ctx.slot_maps[g], cache.k, cache.v, cache.page_size,
                        cache.num_pages, cache.writes)
        ql = ctx.workspace("latent.ql", (T, H * R), self.dtype)
        k.head_product(q, self.w_uk_t, ql)
        ol = ctx.workspace("latent.ol", (T, H * R), self.dtype)
        need = k.attention_scratch_floats(ctx.n_entries, H, R, ctx.max_seq_len, 1, ctx.n_single) if ctx.n_single else 0
        scratch = ctx.workspace("attn.partial", (need,), torch.float32) if need else None
        k.attention(ql, ol, cache.k, cache.v, ctx.block_tables[g], ctx.token_entry, ctx.positions, ctx.q_starts, ctx.seq_lens,
                    H, 1, R, cache.page_size, cache.num_pages, 0, self.scale, scratch, ctx.max_seq_len, ctx.n_single,
                    self._keys_for_the_split(ctx), sink=self.sink)
        o = ctx.workspace("latent.o", (T, self.o_size), self.dtype)
        k.head_product(ol, self.w_uv, o, gate=sums[:, self.q_size + R:] if self.gate else None)
        k.gemm(o, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(o, self.w_o))
        ctx.note_left(h, None)


register_mixer("latent_attention", LatentAttention)

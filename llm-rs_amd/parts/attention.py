"""Causal grouped-query attention over the paged cache.

Parameters: hidden_size, num_heads, num_kv_heads, head_dim, window (None: every
earlier key), position (a position-encoding spec or None), scale (None:
1/sqrt(head_dim), shaders/ops.metal:670), kv_proj (False: the part has no k and
v of its own and only reads a cache that another run wrote).

One step (src/arch/llama.rs:153-163): q, k, v = x Wq^T, x Wk^T, x Wv^T in one
product over the row-concatenated weight; q and k rotated and k, v written into
their pages by the same kernel (for a few tokens) or the next; attention of
every query token over its request's pages; h += o Wo^T with the sum fused into
the product.  No biases.

Options for mixers that prepare q and k otherwise (all off for Llama): `value_dim` (values of another width than
keys), `bias` (q, k and v have biases), `qk_norm_eps` (q and k are divided by their root mean square over the head,
with this eps, no weight), `distance` = "log" (a per-head penalty r1 ln(1 + r2 (i - j)) taken off the scaled score,
with the head's numbers in two tensors), `softcap` (the scaled score s becomes softcap tanh(s / softcap)),
`keep_first` (with a window, the request's first so many keys stay visible at their true positions; their pages stay in
the cache), `o_bias` (the output projection has a bias), `conv` (q, k and v each pass a causal convolution over that many
taps per channel right after the projection, the last tap the current token's, no bias, no activation; the request's
last conv - 1 projected rows are kept in its slot beside the pages), `qk_norm_weight` (the q/k norm multiplies by a
weight of head_dim numbers, one tensor for q and one for k, shared by the heads), a rotation with a `gain` (cosine and
sine both enlarged: the position encoding says so), `gate` = "feature" | "head" (the heads' outputs are multiplied by
sigmoid(Wg x), one gate for every feature of every head or one for each head, before the output projection; the gate's
rows ride in the q/k/v product), `qk_norm_scope` = "projection" (the q/k norm runs over the whole projection, all heads
at once, with a weight of that width, instead of head by head), `value_mix` = "first" | "later" (the values of a
"later" layer become (1 - lambda) v + lambda v_first before they are cached, v_first the values that the "first" such
layer made of the same token in the same step and lambda the layer's one number, tensor leaf `vmix`; the "first" layer
holds the tensor too and does not use it), `names` (the leaves of the tensors' names).  With any of them the q/k/v product leaves
32-bit sums, and one kernel convolves, adds the biases, norms q and k, rotates them (a rotation that the kernels fuse,
angles in 32-bit) and writes k and v into their pages.

The rotation kernels pair neighbours (2i, 2i+1).  Where the encoding pairs
(i, i + rotary_dim/2), the rows of Wq and Wk are reordered within each head at
load so that those two features become neighbours: q.k is a sum over features
and does not care in which order q and k list them, as long as it is the same;
the reference runs files converted for exactly this order (src/arch/llama.rs:156).
"""
from __future__ import annotations

import math

import torch

from ..cache.spec import FixedState, PagedKV
from ..kernels import EPI_ACCUM_F32, EPI_STORE, EPI_STORE_F32, kernels
from .base import Mixer, TensorSpec, build_position, place, register_mixer


class KeyedBySplitChunk:
    """For mixers that call `kernels().attention`: what their recordings are keyed by.  The mixer sets
    `recording_signature = ("attention", kv_heads, head_dim, window)`, the shape of the cache its queries walk."""

    # The kernel library shares the decoding requests' keys out over waves in chunks whose length it chooses by
    # how many keys the step sees (`single_keys`).  A recorded step holds the chunk it was recorded with, so the
    # chunk is part of what recordings are keyed by; and since recording a step again costs about as much as a step
    # while a chunk that is no longer the best one costs a few per cent of the attention, a batch keeps the figure
    # it was recorded with until the rule has asked for another chunk this many steps in a row.
    chunk_patience = 256

    def recording_key(self, ctx):
        k = kernels()
        if not ctx.n_single:
            return 0
        keys = ctx.single_keys(self.recording_signature[3])
        want = k.attention_split_chunk(ctx.n_single, self.recording_signature[1], self.recording_signature[2], ctx.max_seq_len, keys)
        held = ctx.part_state.setdefault(self.recording_signature, {})
        at = (ctx.n_single, ctx.max_seq_len)
        now = held.get(at)             # [chunk, a number of keys that gives it, steps in a row that wanted another, step]
        if now is None or want == now[0] or now[2] >= self.chunk_patience:
            now = held[at] = [want, keys, 0, ctx.serial]
        else:
            now[2] += 1
            now[3] = ctx.serial
        return now[0]

    def _keys_for_the_split(self, ctx) -> int:
        if not ctx.n_single:
            return 0
        now = ctx.part_state.get(self.recording_signature, {}).get((ctx.n_single, ctx.max_seq_len))
        if now is not None and now[3] == ctx.serial:      # this step was keyed by a chunk: the figure that gives it
            return now[1]
        return ctx.single_keys(self.recording_signature[3])


class Attention(KeyedBySplitChunk, Mixer):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.window = int(p.get("window") or 0)
        self.recording_signature = ("attention", self.kv_heads, self.head_dim, self.window)
        self.kv_proj = bool(p.get("kv_proj", True))
        scale = p.get("scale")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.position = build_position(p.get("position"), dtype)
        if self.position is not None and self.position.rotary() is None:
            self.graph_safe = False      # its apply() is free to do anything
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are no multiple of {self.kv_heads} kv heads")
        self.q_size = self.heads * self.head_dim
        self.kv_size = self.kv_heads * self.head_dim
        self.value_dim = int(p.get("value_dim") or self.head_dim)
        self.v_size = self.kv_heads * self.value_dim
        self.o_size = self.heads * self.value_dim
        self.has_bias = bool(p.get("bias", False))
        self.qk_norm_eps = float(p.get("qk_norm_eps") or 0.0)
        self.distance = p.get("distance")
        if self.distance not in (None, "log"):
            raise ValueError(f"unknown distance penalty {self.distance!r} (known: log)")
        self.softcap = float(p.get("softcap") or 0.0)
        self.keep_first = int(p.get("keep_first") or 0) if self.window > 0 else 0
        self.has_o_bias = bool(p.get("o_bias", False))
        if self.softcap < 0 or self.keep_first < 0:
            raise ValueError("softcap and keep_first must not be negative")
        self.taps = int(p.get("conv") or 0)
        self.qk_norm_weight = bool(p.get("qk_norm_weight", False))
        self.gate = p.get("gate")
        if self.gate not in (None, "feature", "head"):
            raise ValueError(f"unknown output gate {self.gate!r} (known: feature, head)")
        if self.qk_norm_weight and not self.qk_norm_eps > 0:
            raise ValueError("a q/k norm with a weight needs its eps (qk_norm_eps)")
        self.norm_whole = p.get("qk_norm_scope", "head") == "projection"
        if p.get("qk_norm_scope", "head") not in ("head", "projection"):
            raise ValueError(f"unknown scope of the q/k norm {p.get('qk_norm_scope')!r} (known: head, projection)")
        if self.norm_whole and not (self.qk_norm_weight and self.kv_proj):
            raise ValueError("a q/k norm over the whole projection has a weight, and keys of the mixer's own")
        self.value_mix = p.get("value_mix")
        if self.value_mix not in (None, "first", "later"):
            raise ValueError(f"unknown part in the mix of values {self.value_mix!r} (known: first, later)")
        if self.value_mix is not None and not self.kv_proj:
            raise ValueError("values that are mixed are the mixer's own")
        if (self.norm_whole or self.value_mix is not None) and (self.taps > 0 or self.has_bias):
            raise ValueError("a q/k norm over the whole projection and a mix of values work on the projection's sums as they are: "
                             "with neither convolutions nor biases")
        if self.taps > 0 and (not self.kv_proj or self.has_bias):
            raise ValueError("convolutions on q, k and v go with neither biases nor a cache that another mixer wrote")
        self.gate_size = {None: 0, "feature": self.o_size, "head": self.heads}[self.gate]
        self.gain = float(getattr(self.position, "gain", 1.0)) if self.position is not None else 1.0
        # q and k are prepared by a kernel of their own between the product and attention
        self.prepared = (self.has_bias or self.qk_norm_eps > 0 or self.distance is not None or self.value_dim != self.head_dim
                         or self.softcap > 0 or self.keep_first > 0 or self.taps > 1 or self.gate is not None or self.gain != 1.0
                         or self.value_mix is not None)
        if self.prepared and self.position is not None and self.position.rotary() is None:
            raise ValueError("a position encoding that is no rotation together with biases, a q/k norm, a distance penalty, a soft cap, "
                             "kept first keys or values of another width is not built")
        leaves = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
                  "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias", "r1": "r1", "r2": "r2",
                  "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "q_conv": "q_conv.weight", "k_conv": "k_conv.weight",
                  "v_conv": "v_conv.weight", "gate": "gate_proj.weight", "value_mix": "vmix", **(p.get("names") or {})}
        self.names = {key: self.name(leaf) for key, leaf in leaves.items()}
        self.w_qkv = None
        self.w_o = None
        self.bias = self.o_bias = self.r1 = self.r2 = None
        self.q_norm = self.k_norm = self.conv = self.mix = None
        # Set by a part that holds this mixer and adds the output projection's bias itself, in a pass over the output
        # that it makes anyway (it reads the bias from `o_bias`): `forward` then leaves the bias out.
        self.output_bias_left_to_holder = False

    def tensors(self):
        n = self.names
        t = {n["q"]: TensorSpec((self.q_size, self.hidden)), n["o"]: TensorSpec((self.hidden, self.o_size))}
        if self.kv_proj:
            t[n["k"]] = TensorSpec((self.kv_size, self.hidden))
            t[n["v"]] = TensorSpec((self.v_size, self.hidden))
        if self.has_bias:
            t[n["q_bias"]] = TensorSpec((self.q_size,))
            if self.kv_proj:
                t[n["k_bias"]] = TensorSpec((self.kv_size,))
                t[n["v_bias"]] = TensorSpec((self.v_size,))
        if self.has_o_bias:
            t[n["o_bias"]] = TensorSpec((self.hidden,))
        if self.distance is not None:
            t[n["r1"]] = TensorSpec((self.heads,), "normal:0.5:0.2")
            t[n["r2"]] = TensorSpec((self.heads,), "normal:0.5:0.05")     # 1 + r2 (i - j) must stay positive
        if self.qk_norm_weight:
            t[n["q_norm"]] = TensorSpec((self.q_size if self.norm_whole else self.head_dim,), "norm")
            if self.kv_proj:
                t[n["k_norm"]] = TensorSpec((self.kv_size if self.norm_whole else self.head_dim,), "norm")
        if self.value_mix is not None:
            t[n["value_mix"]] = TensorSpec((), "normal:0.3:0.1")
        if self.taps > 0:
            t[n["q_conv"]] = TensorSpec((self.q_size, self.taps), "normal:0.0:0.4")
            t[n["k_conv"]] = TensorSpec((self.kv_size, self.taps), "normal:0.0:0.4")
            t[n["v_conv"]] = TensorSpec((self.v_size, self.taps), "normal:0.0:0.4")
        if self.gate is not None:
            t[n["gate"]] = TensorSpec((self.gate_size, self.hidden))
        return t

    def _pair_neighbours(self, w: torch.Tensor, heads: int, undo: bool = False) -> torch.Tensor:
        """Rows of a q or k weight reordered so that each rotation pair is (2i, 2i+1); `undo` puts them back."""
        rotary = self.position.rotary() if self.position is not None else None
        if rotary is None or rotary[2] or rotary[1] == 0:
            return w          # no rotation here, or the pairs are neighbours already
        rot = rotary[1]
        order = torch.stack([torch.arange(rot // 2), torch.arange(rot // 2) + rot // 2], dim=1).flatten()
        order = torch.cat([order, torch.arange(rot, self.head_dim)])
        if undo:
            order = torch.argsort(order)
        return w.view(heads, self.head_dim, -1)[:, order.to(w.device), :].reshape(w.shape)

    def load(self, tensors, device):
        get = lambda n: place(tensors[self.names[n]], device, self.dtype)
        get32 = lambda n: place(tensors[self.names[n]], device, torch.float32)
        parts = [self._pair_neighbours(get("q"), self.heads)]
        if self.kv_proj:
            parts += [self._pair_neighbours(get("k"), self.kv_heads), get("v")]
        self.qkv_width = sum(w.shape[0] for w in parts)
        if self.gate is not None:       # the gate's rows behind q | k | v: one product for all that reads the mixer's input
            parts.append(get("gate"))
        self.w_qkv = torch.cat(parts, dim=0).contiguous()
        self.w_o = get("o")
        if self.qk_norm_weight:         # (a head's features are listed in the order its rotation pairs them in)
            hq, hk = (self.heads, self.kv_heads) if self.norm_whole else (1, 1)
            self.q_norm = self._pair_neighbours(get32("q_norm").unsqueeze(1), hq).squeeze(1).contiguous()
            self.k_norm = self._pair_neighbours(get32("k_norm").unsqueeze(1), hk).squeeze(1).contiguous() if self.kv_proj else None
        if self.value_mix is not None:
            self.mix = get32("value_mix").reshape(1)        # stays on the device: the kernel reads it there
        if self.taps > 0:               # the taps of q | k | v one under the other, as the product's columns are
            self.conv = torch.cat([self._pair_neighbours(get32("q_conv"), self.heads), self._pair_neighbours(get32("k_conv"), self.kv_heads),
                                   get32("v_conv")], dim=0).contiguous()
        if self.has_bias:       # added to the 32-bit sums: kept in 32-bit, side by side as the product's columns are (and reordered as its rows are)
            pair = lambda b, heads: self._pair_neighbours(b.unsqueeze(1), heads).squeeze(1)
            self.bias = torch.cat([pair(get32("q_bias"), self.heads)] +
                                  ([pair(get32("k_bias"), self.kv_heads), get32("v_bias")] if self.kv_proj else [])).contiguous()
        if self.has_o_bias:
            self.o_bias = get32("o_bias")
        if self.distance is not None:
            self.r1, self.r2 = get32("r1"), get32("r2")
        if self.position is not None:
            self.position.to(device)

    def export(self):
        w = self.w_qkv.cpu()
        n = self.names
        out = {n["q"]: self._pair_neighbours(w[:self.q_size], self.heads, undo=True).contiguous(), n["o"]: self.w_o.cpu()}
        if self.gate is not None:
            out[n["gate"]] = w[self.qkv_width:].contiguous()
        if self.qk_norm_weight:
            hq, hk = (self.heads, self.kv_heads) if self.norm_whole else (1, 1)
            out[n["q_norm"]] = self._pair_neighbours(self.q_norm.cpu().unsqueeze(1), hq, undo=True).squeeze(1).contiguous()
            if self.kv_proj:
                out[n["k_norm"]] = self._pair_neighbours(self.k_norm.cpu().unsqueeze(1), hk, undo=True).squeeze(1).contiguous()
        if self.value_mix is not None:
            out[n["value_mix"]] = self.mix.cpu().reshape(())
        if self.taps > 0:
            c = self.conv.cpu()
            out[n["q_conv"]] = self._pair_neighbours(c[:self.q_size], self.heads, undo=True).contiguous()
            out[n["k_conv"]] = self._pair_neighbours(c[self.q_size:self.q_size + self.kv_size], self.kv_heads, undo=True).contiguous()
            out[n["v_conv"]] = c[self.q_size + self.kv_size:].contiguous()
        if self.kv_proj:
            k, v = w[self.q_size:self.q_size + self.kv_size], w[self.q_size + self.kv_size:self.qkv_width]
            out[n["k"]] = self._pair_neighbours(k, self.kv_heads, undo=True).contiguous()
            out[n["v"]] = v.contiguous()
        if self.has_bias:
            b = self.bias.cpu()
            unpair = lambda x, heads: self._pair_neighbours(x.unsqueeze(1), heads, undo=True).squeeze(1).contiguous()
            out[n["q_bias"]] = unpair(b[:self.q_size], self.heads)
            if self.kv_proj:
                out[n["k_bias"]] = unpair(b[self.q_size:self.q_size + self.kv_size], self.kv_heads)
                out[n["v_bias"]] = b[self.q_size + self.kv_size:].contiguous()
        if self.has_o_bias:
            out[n["o_bias"]] = self.o_bias.cpu()
        if self.distance is not None:
            out[n["r1"]], out[n["r2"]] = self.r1.cpu(), self.r2.cpu()
        return out

    def cache_need(self):
        pages = PagedKV(self.kv_heads, self.head_dim, self.window, self.value_dim if self.value_dim != self.head_dim else 0, self.keep_first)
        if self.taps > 1:       # beside the pages, in the request's slot: the last conv - 1 rows of q | k | v as projected, 32-bit
            return (pages, FixedState(((self.taps - 1) * self.qkv_columns,), torch.float32))
        return pages

    @property
    def qkv_columns(self) -> int:
        return self.q_size + (self.kv_size + self.v_size if self.kv_proj else 0)

    def _forward_prepared(self, ctx, x, h, cache):
        """The product's 32-bit sums -> convolution, biases, norm and rotation of q and k, cache write -> attention with
        the distance penalty, the soft cap, the kept first keys and the output gate (applied to the 32-bit results on their
        way out) -> the output projection."""
        k = kernels()
        T = x.shape[0]
        conv_state = None
        if cache.kind == "several":          # pages, and the convolutions' last inputs in the request's slot
            cache, conv_state = cache.parts[0], cache.parts[1].state
        write = self.kv_proj and cache.writes
        n_kv = self.kv_heads if self.kv_proj else 0
        g = cache.group
        C = self.qkv_columns
        sums = ctx.workspace("attn.sums", (T, self.w_qkv.shape[0]), torch.float32)
        k.gemm(x, self.w_qkv, sums, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_qkv))
        eps, q_weight, k_weight = self.qk_norm_eps, self.q_norm, self.k_norm
        if self.norm_whole or self.value_mix is not None:
            # the norms over the whole projection and the mix of the values, in place on the sums; the first mixing
            # layer's values stay in a buffer of their own for the later ones of the step
            first = ctx.workspace("attn.value_first", (T, self.v_size), torch.float32) if self.value_mix is not None else None
            k.qkv_whole(sums, self.q_size, self.kv_size, self.v_size, q_weight if self.norm_whole else None,
                        k_weight if self.norm_whole else None, eps, first=first if self.value_mix == "later" else None,
                        lam=self.mix if self.value_mix == "later" else None, keep=first if self.value_mix == "first" else None)
            if self.norm_whole:
                eps, q_weight, k_weight = 0.0, None, None
        q = ctx.workspace("attn.qkv", (T, self.q_size), self.dtype)
        rotary = self.position.rotary() if self.position is not None else None
        inv_freq, rotary_dim = (None, 0) if rotary is None else rotary[:2]
        # (one tap: every channel times its number, and nothing to remember)
        conv = (self.conv, conv_state, ctx.q_starts, ctx.slots, ctx.token_entry) if self.taps > 0 else None
        k.qkv_finish(sums[:, :C], self.bias, q, ctx.slot_maps[g], cache.k, cache.v, self.heads, n_kv, self.head_dim, self.value_dim,
                     cache.page_size, cache.num_pages, write, eps, ctx.positions, inv_freq, rotary_dim,
                     q_weight=q_weight, k_weight=k_weight, gain=self.gain, conv=conv)
        if self.taps > 1:
            k.conv_state_update(sums[:, :C], conv_state, ctx.q_starts, ctx.slots, C, self.taps)
        o = ctx.workspace("attn.out", (T, self.o_size), self.dtype)
        need = k.attention_scratch_floats(ctx.n_entries, self.heads, max(self.head_dim, self.value_dim), ctx.max_seq_len,
                                          self.kv_heads, ctx.n_single) if ctx.n_single else 0
        scratch = ctx.workspace("attn.partial", (need,), torch.float32) if need else None
        k.attention(q, o, cache.k, cache.v, ctx.block_tables[g], ctx.token_entry, ctx.positions, ctx.q_starts, ctx.seq_lens,
                    self.heads, self.kv_heads, self.head_dim, cache.page_size, cache.num_pages, self.window, self.scale,
                    scratch, ctx.max_seq_len, ctx.n_single, self._keys_for_the_split(ctx), value_dim=self.value_dim,
                    distance=None if self.distance is None else (self.r1, self.r2), softcap=self.softcap, keep_first=self.keep_first,
                    gate=sums[:, self.qkv_width:] if self.gate is not None else None, gate_per=1 if self.gate == "feature" else self.value_dim)
        k.gemm(o, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(o, self.w_o))
        if self.has_o_bias and not self.output_bias_left_to_holder:
            k.add_bias_rows(h, self.o_bias)
        ctx.note_left(h, None)

    def takes_normed_rows(self, ctx, rows):
        if self.prepared:
            return False
        # the q/k/v product norms its rows itself where it is the fused kernel: a rotation it applies (or none)
        fused = self.position is None or self.position.rotary() is not None
        return fused and kernels().product_norms_its_rows(rows, self.w_qkv.shape[0], self.hidden, self.dtype)

    def forward(self, ctx, x, h, cache):
        if self.prepared:
            return self._forward_prepared(ctx, x, h, cache)
        k = kernels()
        T = x.shape[0]
        write = self.kv_proj and cache.writes
        n_kv = self.kv_heads if self.kv_proj else 0
        qkv = ctx.workspace("attn.qkv", (T, self.q_size + 2 * n_kv * self.head_dim), self.dtype)
        rotary = self.position.rotary() if self.position is not None else None
        g = cache.group
        if self.position is None or rotary is not None:
            inv_freq, rotary_dim = (None, 0) if rotary is None else rotary[:2]
            k.qkv_rope_cache(x, self.w_qkv, qkv, ctx.positions, ctx.slot_maps[g], inv_freq, rotary_dim, cache.k, cache.v,
                             self.heads, n_kv, self.head_dim, cache.page_size, cache.num_pages, write,
                             ctx.gemm_workspace(x, self.w_qkv))
        else:     # an encoding of its own: it changes q and k between the product and the cache write
            k.gemm(x, self.w_qkv, qkv, EPI_STORE, ctx.gemm_workspace(x, self.w_qkv))
            q3 = qkv[:, :self.q_size].unflatten(1, (self.heads, self.head_dim))
            k3 = qkv[:, self.q_size:self.q_size + self.kv_size].unflatten(1, (self.kv_heads, self.head_dim)) if n_kv else None
            self.position.apply(ctx, q3, k3)
            if write:
                k.rope_kv_write(qkv, ctx.positions, ctx.slot_maps[g], None, 0, False, cache.k, cache.v,
                                self.heads, n_kv, self.head_dim, cache.page_size, cache.num_pages, write)
        o = ctx.workspace("attn.out", (T, self.q_size), self.dtype)
        # room for the partial results of single-token entries, which the kernel splits by key range
        need = k.attention_scratch_floats(ctx.n_entries, self.heads, self.head_dim, ctx.max_seq_len, self.kv_heads, ctx.n_single) if ctx.n_single else 0
        scratch = ctx.workspace("attn.partial", (need,), torch.float32) if need else None
        k.attention(qkv[:, :self.q_size], o, cache.k, cache.v, ctx.block_tables[g], ctx.token_entry, ctx.positions,
                    ctx.q_starts, ctx.seq_lens, self.heads, self.kv_heads, self.head_dim, cache.page_size,
                    cache.num_pages, self.window, self.scale, scratch, ctx.max_seq_len, ctx.n_single,
                    self._keys_for_the_split(ctx))
        leave = ctx.room_for_next_norm(h, self.w_o) if not self.has_o_bias else None
        k.gemm(o, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(o, self.w_o), **({} if leave is None else {"leave": leave}))
        if self.has_o_bias and not self.output_bias_left_to_holder:
            k.add_bias_rows(h, self.o_bias)
        ctx.note_left(h, leave)


register_mixer("attention", Attention)

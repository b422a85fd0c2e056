"""Mixers that keep a matrix per head as their memory, S [key channel, value channel] in 32-bit in the request's slot,
and the mixer that runs several mixers side by side.

"lightning"(hidden_size, heads, dim, vdim, decay[heads], eps): linear attention with a fixed decay per head.
q, k = silu(Wq x), silu(Wk x) [heads, dim]; v = silu(Wv x) [heads, vdim]; S_t = decay_h S_(t-1) + k_t v_t^T;
o_t = S_t^T q_t; the heads side by side are RMS-normed together (weight `norm`), times sigmoid(Wg x), through Wo.
One product gives q | k | v | gate as 32-bit sums; the recurrence and everything after it are 32-bit up to Wo's input.

"delta_rule"(hidden_size, heads, kv_heads, dim, vdim, conv, eps, unit_eps, decay_rank, gate_rank): the gated delta
rule.  q, k [kv_heads, dim] and v [heads, vdim] each pass a causal convolution over `conv` taps (the last tap the
current token's, no bias) and silu; q and k become unit vectors per head (x / sqrt(sum x^2 + unit_eps)), q times
dim^(-1/2); beta = sigmoid(Wb x) per head; a decay per head and key channel g = exp(-exp(A_log_h) softplus(Wa2 Wa1 x +
dt_bias)); S <- g S (rows); u = beta (v - S^T k); S <- S + k u^T; o = S^T q; each head's o is RMS-normed over vdim
(weight `norm` [vdim], the same for every head), times sigmoid(Wg2 Wg1 x), through Wo.  The request's state is S and
the convolutions' last conv - 1 inputs.

"mlstm"(hidden_size, heads, dim, vdim, gate_cap, eps): a matrix memory with exponential gates.  q = Wq x dim^(-1/2),
k = Wk x [heads, dim], v = Wv x [heads, vdim]; per head the logarithms of an input and a forget gate,
i = cap tanh((Wi x + bi) / cap), f = log sigmoid(cap tanh((Wf x + bf) / cap)); a running maximum m_t = max(f + m_(t-1), i)
(m_0 = 0) keeps the exponentials in range: S_t = exp(f + m_(t-1) - m_t) S_(t-1) + exp(i - m_t) k v^T, n_t the same with k
alone, o = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6); each head's o is RMS-normed, the heads side by side times the
weight `norm`, times sigmoid(Wg x), through Wo.  The request's state is S, n and m.  n is kept as one more column of S:
the recurrence writes a 1 in the value's place there, so S^T q also yields n . q.

"parallel"(hidden_size, eps, branches = [{name, mixer: PartSpec-like, out: leaf of the branch's output norm}]): every
branch reads the same input; the result is the mean of the branches' outputs, each RMS-normed over the model width with
a weight of its own.  The branches are mixers of any registered kind, each with the cache it asks for.
"""
from __future__ import annotations

import torch

from ..cache.spec import FixedState
from ..config.spec import PartSpec
from ..kernels import EPI_ACCUM_F32, EPI_STORE, EPI_STORE_F32, kernels
from .base import Mixer, TensorSpec, build_mixer, place, register_mixer


def _leaves(defaults: dict, given) -> dict:
    return {**defaults, **(given or {})}


class Lightning(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.heads, self.dk, self.dv = int(p["hidden_size"]), int(p["heads"]), int(p["dim"]), int(p["vdim"])
        self.eps = float(p["eps"])
        self.decay_values = [float(d) for d in p["decay"]]
        if len(self.decay_values) != self.heads:
            raise ValueError(f"{len(self.decay_values)} decays for {self.heads} heads")
        leaves = _leaves({"q": "q", "k": "k", "v": "v", "gate": "g", "out": "o", "norm": "norm"}, p.get("names"))
        self.names = {k: self.name(v) for k, v in leaves.items()}
        self.qk, self.vw = self.heads * self.dk, self.heads * self.dv
        self.w_in = self.w_o = self.norm = self.decay = None

    def tensors(self):
        n, H = self.names, self.hidden
        return {n["q"]: TensorSpec((self.qk, H)), n["k"]: TensorSpec((self.qk, H)), n["v"]: TensorSpec((self.vw, H)),
                n["gate"]: TensorSpec((self.vw, H)), n["out"]: TensorSpec((H, self.vw)), n["norm"]: TensorSpec((self.vw,), "norm")}

    def load(self, tensors, device):
        n = self.names
        get = lambda key: place(tensors[n[key]], device, self.dtype)
        self.w_in = torch.cat([get("q"), get("k"), get("v"), get("gate")], dim=0).contiguous()
        self.w_o = get("out")
        self.norm = place(tensors[n["norm"]], device, torch.float32)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(device)

    def export(self):
        n, w = self.names, self.w_in.cpu()
        a, b, c = self.qk, 2 * self.qk, 2 * self.qk + self.vw
        return {n["q"]: w[:a].contiguous(), n["k"]: w[a:b].contiguous(), n["v"]: w[b:c].contiguous(), n["gate"]: w[c:].contiguous(),
                n["out"]: self.w_o.cpu(), n["norm"]: self.norm.cpu()}

    def cache_need(self):
        return FixedState((self.heads * self.dk * self.dv,), torch.float32)

    def forward(self, ctx, x, h, cache):
        k = kernels()
        T = x.shape[0]
        a, b, c = self.qk, 2 * self.qk, 2 * self.qk + self.vw
        sums = ctx.workspace("linear.sums", (T, c + self.vw), torch.float32)
        k.gemm(x, self.w_in, sums, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_in))
        k.silu_columns(sums, 0, c)
        o = ctx.workspace("linear.o", (T, self.vw), torch.float32)
        k.linear_scan(sums[:, :a], sums[:, a:b], sums[:, b:c], cache.state, ctx.q_starts, ctx.slots, self.heads, self.heads,
                      self.dk, self.dv, o, decay=self.decay)
        gated = ctx.workspace("linear.gated", (T, self.vw), self.dtype)
        k.gated_rmsnorm(gated, o, sums[:, c:], self.norm, self.vw, self.eps)
        k.gemm(gated, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(gated, self.w_o))
        ctx.note_left(h, None)


class DeltaRule(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.heads, self.kv_heads = int(p["hidden_size"]), int(p["heads"]), int(p["kv_heads"])
        self.dk, self.dv, self.taps = int(p["dim"]), int(p["vdim"]), int(p["conv"])
        self.eps, self.unit_eps = float(p["eps"]), float(p.get("unit_eps", 1e-6))
        self.decay_rank, self.gate_rank = int(p["decay_rank"]), int(p["gate_rank"])
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are no multiple of {self.kv_heads} q/k heads")
        if self.taps < 1:
            raise ValueError("the convolution has at least one tap")
        leaves = _leaves({"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "beta": "b",
                          "A_log": "A_log", "dt_bias": "dt_bias", "a1": "a1", "a2": "a2", "g1": "g1", "g2": "g2", "norm": "norm",
                          "out": "o"}, p.get("names"))
        self.names = {k: self.name(v) for k, v in leaves.items()}
        self.qk, self.vw, self.gw = self.kv_heads * self.dk, self.heads * self.dv, self.heads * self.dk
        self.channels = 2 * self.qk + self.vw          # what passes the convolutions: q | k | v
        self.w_in = self.w_low = self.w_a2 = self.w_g2 = self.w_o = None
        self.conv = self.A_log = self.dt_bias = self.norm = None

    def tensors(self):
        n, H = self.names, self.hidden
        return {n["q"]: TensorSpec((self.qk, H)), n["k"]: TensorSpec((self.qk, H)), n["v"]: TensorSpec((self.vw, H)),
                n["q_conv"]: TensorSpec((self.qk, self.taps), "normal:0.0:0.3"), n["k_conv"]: TensorSpec((self.qk, self.taps), "normal:0.0:0.3"),
                n["v_conv"]: TensorSpec((self.vw, self.taps), "normal:0.0:0.3"), n["beta"]: TensorSpec((self.heads, H)),
                n["A_log"]: TensorSpec((self.heads,), "normal:0.0:0.5"), n["dt_bias"]: TensorSpec((self.gw,), "normal:-1.0:0.5"),
                n["a1"]: TensorSpec((self.decay_rank, H)), n["a2"]: TensorSpec((self.gw, self.decay_rank), "normal:0.0:0.1"),
                n["g1"]: TensorSpec((self.gate_rank, H)), n["g2"]: TensorSpec((self.vw, self.gate_rank), "normal:0.0:0.1"),
                n["norm"]: TensorSpec((self.dv,), "norm"), n["out"]: TensorSpec((H, self.vw))}

    def load(self, tensors, device):
        n = self.names
        get = lambda key: place(tensors[n[key]], device, self.dtype)
        get32 = lambda key: place(tensors[n[key]], device, torch.float32)
        # one product for what enters the recurrence in 32-bit (q | k | v | beta), one for the two narrow projections
        # whose outputs are the next products' inputs (a1 | g1)
        self.w_in = torch.cat([get("q"), get("k"), get("v"), get("beta")], dim=0).contiguous()
        self.w_low = torch.cat([get("a1"), get("g1")], dim=0).contiguous()
        self.w_a2, self.w_g2, self.w_o = get("a2"), get("g2"), get("out")
        self.conv = torch.cat([get32("q_conv"), get32("k_conv"), get32("v_conv")], dim=0).contiguous()
        self.A_log, self.dt_bias, self.norm = get32("A_log"), get32("dt_bias"), get32("norm")

    def export(self):
        n, w, low, conv = self.names, self.w_in.cpu(), self.w_low.cpu(), self.conv.cpu()
        a, b, c = self.qk, 2 * self.qk, self.channels
        return {n["q"]: w[:a].contiguous(), n["k"]: w[a:b].contiguous(), n["v"]: w[b:c].contiguous(), n["beta"]: w[c:].contiguous(),
                n["a1"]: low[:self.decay_rank].contiguous(), n["g1"]: low[self.decay_rank:].contiguous(),
                n["a2"]: self.w_a2.cpu(), n["g2"]: self.w_g2.cpu(), n["out"]: self.w_o.cpu(),
                n["q_conv"]: conv[:a].contiguous(), n["k_conv"]: conv[a:b].contiguous(), n["v_conv"]: conv[b:].contiguous(),
                n["A_log"]: self.A_log.cpu(), n["dt_bias"]: self.dt_bias.cpu(), n["norm"]: self.norm.cpu()}

    def cache_need(self):
        # one row per request: S [heads, dim, vdim], then the convolutions' last inputs [conv - 1, channels]
        return FixedState((self.heads * self.dk * self.dv + (self.taps - 1) * self.channels,), torch.float32)

    def forward(self, ctx, x, h, cache):
        k = kernels()
        T, C = x.shape[0], self.channels
        a, b = self.qk, 2 * self.qk
        n_state = self.heads * self.dk * self.dv
        sums = ctx.workspace("delta.sums", (T, C + self.heads), torch.float32)
        k.gemm(x, self.w_in, sums, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_in))
        low = ctx.workspace("delta.low", (T, self.decay_rank + self.gate_rank), self.dtype)
        k.gemm(x, self.w_low, low, EPI_STORE, ctx.gemm_workspace(x, self.w_low))
        decay = ctx.workspace("delta.decay", (T, self.gw), torch.float32)
        low_a, low_g = low[:, :self.decay_rank], low[:, self.decay_rank:]
        k.gemm(low_a, self.w_a2, decay, EPI_STORE_F32, ctx.gemm_workspace(low_a, self.w_a2))
        gate = ctx.workspace("delta.gate", (T, self.vw), torch.float32)
        k.gemm(low_g, self.w_g2, gate, EPI_STORE_F32, ctx.gemm_workspace(low_g, self.w_g2))
        qkv = ctx.workspace("delta.qkv", (T, C), torch.float32)
        k.causal_conv_silu(sums, self.conv, None, cache.state[:, n_state:], ctx.q_starts, ctx.slots, ctx.token_entry, C, qkv)
        beta = sums[:, C:]
        k.delta_prepare(qkv[:, :a], qkv[:, a:b], decay, beta, self.A_log, self.dt_bias, self.heads, self.kv_heads, self.dk, self.unit_eps)
        o = ctx.workspace("delta.o", (T, self.vw), torch.float32)
        k.linear_scan(qkv[:, :a], qkv[:, a:b], qkv[:, b:], cache.state[:, :n_state], ctx.q_starts, ctx.slots, self.heads, self.kv_heads,
                      self.dk, self.dv, o, g=decay, beta=beta)
        gated = ctx.workspace("delta.gated", (T, self.vw), self.dtype)
        k.gated_rmsnorm(gated, o, gate, self.norm, self.dv, self.eps)
        k.gemm(gated, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(gated, self.w_o))
        ctx.note_left(h, None)


class MLSTM(Mixer):
    graph_safe = True
    DEN_ADD = 1e-6          # what the read-out's denominator is enlarged by

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.heads, self.dk, self.dv = int(p["hidden_size"]), int(p["heads"]), int(p["dim"]), int(p["vdim"])
        self.cap, self.eps = float(p["gate_cap"]), float(p["eps"])
        if not self.cap > 0:
            raise ValueError(f"the gates' cap must be positive, got {self.cap}")
        leaves = _leaves({"q": "q", "k": "k", "v": "v", "gate": "g", "out": "o", "norm": "norm", "i": "i", "i_bias": "i.b", "f": "f",
                          "f_bias": "f.b"}, p.get("names"))
        self.names = {k: self.name(v) for k, v in leaves.items()}
        self.qk, self.vw = self.heads * self.dk, self.heads * self.dv
        self.cols = self.dv + 1                           # a head's columns of S: its value channels, then n
        self.n_matrix = self.heads * self.cols * self.dk  # floats of S and n in a request's state; the maxima follow
        self.w_in = self.w_o = self.norm = self.bias_i = self.bias_f = None

    def tensors(self):
        n, H = self.names, self.hidden
        return {n["q"]: TensorSpec((self.qk, H)), n["k"]: TensorSpec((self.qk, H)), n["v"]: TensorSpec((self.vw, H)),
                n["gate"]: TensorSpec((self.vw, H)), n["out"]: TensorSpec((H, self.vw)), n["norm"]: TensorSpec((self.vw,), "norm"),
                n["i"]: TensorSpec((self.heads, H), "normal:0.0:0.1"), n["i_bias"]: TensorSpec((self.heads,), "normal:0.0:0.5"),
                n["f"]: TensorSpec((self.heads, H), "normal:0.0:0.1"), n["f_bias"]: TensorSpec((self.heads,), "normal:3.0:1.0")}

    def load(self, tensors, device):
        n = self.names
        get = lambda key: place(tensors[n[key]], device, self.dtype)
        # one product for everything that reads the mixer's input, left as 32-bit sums: q | k | v | gate | i | f
        self.w_in = torch.cat([get("q"), get("k"), get("v"), get("gate"), get("i"), get("f")], dim=0).contiguous()
        self.w_o = get("out")
        self.norm = place(tensors[n["norm"]], device, torch.float32)
        self.bias_i = place(tensors[n["i_bias"]], device, torch.float32)
        self.bias_f = place(tensors[n["f_bias"]], device, torch.float32)

    def export(self):
        n, w = self.names, self.w_in.cpu()
        a, b, c, d, e = self.qk, 2 * self.qk, 2 * self.qk + self.vw, 2 * self.qk + 2 * self.vw, 2 * self.qk + 2 * self.vw + self.heads
        return {n["q"]: w[:a].contiguous(), n["k"]: w[a:b].contiguous(), n["v"]: w[b:c].contiguous(), n["gate"]: w[c:d].contiguous(),
                n["i"]: w[d:e].contiguous(), n["f"]: w[e:].contiguous(), n["out"]: self.w_o.cpu(), n["norm"]: self.norm.cpu(),
                n["i_bias"]: self.bias_i.cpu(), n["f_bias"]: self.bias_f.cpu()}

    def cache_need(self):
        # one row per request, zero at its start: S with n as its last column [heads, vdim + 1, dim], then m [heads]
        # (in room for a multiple of four, so that a slot's rows stay whole 16-byte pieces where S's are)
        return FixedState((self.n_matrix + -(-self.heads // 4) * 4,), torch.float32)

    def forward(self, ctx, x, h, cache):
        k = kernels()
        T, H = x.shape[0], self.heads
        a, b, c, d = self.qk, 2 * self.qk, 2 * self.qk + self.vw, 2 * self.qk + 2 * self.vw
        sums = ctx.workspace("linear.sums", (T, d + 2 * H), torch.float32)
        k.gemm(x, self.w_in, sums, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_in))
        gates = ctx.workspace("mlstm.gates", (3, T, H), torch.float32)          # decay, take, floor
        k.exp_gates(sums[:, d:d + H], sums[:, d + H:], self.bias_i, self.bias_f, self.cap, cache.state[:, self.n_matrix:],
                    ctx.q_starts, ctx.slots, gates[0], gates[1], gates[2])
        o = ctx.workspace("mlstm.o", (T, H * self.cols), torch.float32)
        k.linear_scan(sums[:, :a], sums[:, a:b], sums[:, b:c], cache.state[:, :self.n_matrix], ctx.q_starts, ctx.slots, H, H,
                      self.dk, self.cols, o, gates=(gates[0], gates[1]), v_cols=self.dv)
        gated = ctx.workspace("linear.gated", (T, self.vw), self.dtype)
        # (q's factor dim^(-1/2) multiplies the read-out and its normaliser alike: applied here, to both)
        k.gated_rmsnorm(gated, o, sums[:, c:d], self.norm, self.dv, self.eps, floor=gates[2], x_scale=self.dk ** -0.5, den_add=self.DEN_ADD)
        k.gemm(gated, self.w_o, h, EPI_ACCUM_F32, ctx.gemm_workspace(gated, self.w_o))
        ctx.note_left(h, None)


class Parallel(Mixer):
    """Branches side by side on the same input; h += mean_b rmsnorm(branch_b(x)) * out_b."""

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.eps = int(p["hidden_size"]), float(p["eps"])
        self.branches = []          # (mixer, full name of its output norm's weight)
        for br in p["branches"]:
            sub = br["mixer"]
            if not isinstance(sub, PartSpec):
                sub = PartSpec(sub["kind"], sub.get("prefix", ""), sub.get("params", {}))
            self.branches.append((build_mixer(sub, dtype), self.name(br["out"])))
        if not 1 <= len(self.branches) <= 2:
            raise ValueError("one or two mixers side by side")
        self.graph_safe = all(m.graph_safe for m, _ in self.branches)
        keyed = [m for m, _ in self.branches if m.recording_signature is not None]
        self._keyed = keyed
        self.recording_signature = tuple(m.recording_signature for m in keyed) or None
        self.out_weights, self.out_biases = [], []
        # the branches' needs, in their order; a branch without a need has no part in the view
        self._needs = [m.cache_need() for m, _ in self.branches]

    def recording_key(self, ctx):
        return tuple(m.recording_key(ctx) for m in self._keyed)

    def tensors(self):
        t = {}
        for m, out in self.branches:
            t.update(m.tensors())
            t[out] = TensorSpec((self.hidden,), "norm")
        return t

    def load(self, tensors, device):
        self.out_weights, self.out_biases = [], []
        for m, out in self.branches:
            m.load(tensors, device)
            self.out_weights.append(place(tensors[out], device, torch.float32))
            # a branch whose output projection has a bias leaves it to the kernel that norms the branches' outputs
            bias = getattr(m, "o_bias", None) if hasattr(m, "output_bias_left_to_holder") else None
            if bias is not None:
                m.output_bias_left_to_holder = True
            self.out_biases.append(bias)

    def export(self):
        t = {}
        for (m, out), w in zip(self.branches, self.out_weights):
            t.update(m.export())
            t[out] = w.cpu()
        return t

    def step_weight_bytes(self, seen):
        total = sum(m.step_weight_bytes(seen) for m, _ in self.branches)
        return total + sum(w.numel() * 4 for w in self.out_weights)

    def cache_need(self):
        return tuple(n for n in self._needs if n is not None)

    def forward(self, ctx, x, h, cache):
        k = kernels()
        T = x.shape[0]
        ys = ctx.workspace("parallel.y", (len(self.branches), T, self.hidden), torch.float32)
        ys.zero_()                                   # (a fill kernel: the branches add their results into it)
        views = iter(cache.parts)
        for i, (m, _) in enumerate(self.branches):
            m.forward(ctx, x, ys[i], next(views) if self._needs[i] is not None else None)
        k.rmsnorm_sum(h, [(ys[i], b, w) for i, (w, b) in enumerate(zip(self.out_weights, self.out_biases))], 1.0 / len(self.branches), self.eps)
        ctx.note_left(h, None)


register_mixer("lightning", Lightning)
register_mixer("delta_rule", DeltaRule)
register_mixer("mlstm", MLSTM)
register_mixer("parallel", Parallel)

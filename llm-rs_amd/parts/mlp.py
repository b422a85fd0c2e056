"""SwiGLU feed-forward(hidden_size, intermediate_size):
h += (silu(x Wg^T) * (x Wu^T)) Wd^T, silu(v) = v / (1 + exp(-v))
(src/arch/llama.rs:165-170, shaders/ops.metal:762-793).  The gate and up weights
are interleaved row by row at load, so one product yields (gate_j, up_j) side by
side and its epilogue writes silu(gate) * up, computed in 32-bit, once; the down
product adds into the 32-bit residual stream.  No biases."""
from __future__ import annotations

import contextlib

import torch

from ..kernels import EPI_ACCUM_F32, EPI_GLU_CLAMP, EPI_STORE_F32, EPI_SWIGLU, KernelError, kernels, stand_in_kernels
from .base import FeedForward, TensorSpec, build_feed_forward, place, register_feed_forward


class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        # the leaves of the three tensors' names, for files that call them otherwise: {"gate": ..., "up": ..., "down": ...}
        leaves = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight", **(spec.params.get("names") or {})}
        self.n_gate, self.n_up, self.n_down = (self.name(leaves[k]) for k in ("gate", "up", "down"))
        self.w_gate_up = None
        self.w_down = None

    def tensors(self):
        return {self.n_gate: TensorSpec((self.inter, self.hidden)),
                self.n_up: TensorSpec((self.inter, self.hidden)),
                self.n_down: TensorSpec((self.hidden, self.inter))}

    def load(self, tensors, device):
        gate = place(tensors[self.n_gate], device, self.dtype)
        up = place(tensors[self.n_up], device, self.dtype)
        self.w_gate_up = torch.stack([gate, up], dim=1).reshape(2 * self.inter, self.hidden).contiguous()
        self.w_down = place(tensors[self.n_down], device, self.dtype)

    def export(self):
        both = self.w_gate_up.cpu().view(self.inter, 2, self.hidden)
        return {self.n_gate: both[:, 0, :].contiguous(), self.n_up: both[:, 1, :].contiguous(),
                self.n_down: self.w_down.cpu()}

    def takes_normed_rows(self, ctx, rows):
        return kernels().product_norms_its_rows(rows, 2 * self.inter, self.hidden, self.dtype)

    def forward(self, ctx, x, h):
        k = kernels()
        act = ctx.workspace("mlp.act", (x.shape[0], self.inter), self.dtype)
        k.gemm(x, self.w_gate_up, act, EPI_SWIGLU, ctx.gemm_workspace(x, self.w_gate_up))
        leave = ctx.room_for_next_norm(h, self.w_down)
        k.gemm(act, self.w_down, h, EPI_ACCUM_F32, ctx.gemm_workspace(act, self.w_down), **({} if leave is None else {"leave": leave}))
        ctx.note_left(h, leave)


register_feed_forward("swiglu", SwiGLU)


ACTIVATIONS = ("relu2", "clamped_glu")       # relu(x)^2; gated: g sigmoid(alpha g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit)
GATED = ("clamped_glu",)                     # activations of two projections, gate and up


class ClampedGLU(FeedForward):
    """Feed-forward with a clamped, gated activation(hidden_size, intermediate_size, limit, alpha):
    h += Wdown (g sigmoid(alpha g) (u + 1)), g = min(Wgate x, limit), u = clamp(Wup x, -limit, limit); alpha is 1.702
    unless given.  The gate and up weights are interleaved row by row at load, so one product yields (gate_j, up_j) side
    by side and its epilogue writes the activation, computed on the 32-bit sums and rounded once; the down product adds
    into the 32-bit stream."""
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.limit, self.alpha = float(p["limit"]), float(p.get("alpha", 1.702))
        if not self.limit > 0:
            raise ValueError(f"the activation's limit must be positive, got {self.limit}")
        leaves = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight", **(p.get("names") or {})}
        self.n_gate, self.n_up, self.n_down = (self.name(leaves[k]) for k in ("gate", "up", "down"))
        self.w_gate_up = self.w_down = self.glu = None

    def tensors(self):
        return {self.n_gate: TensorSpec((self.inter, self.hidden)), self.n_up: TensorSpec((self.inter, self.hidden)),
                self.n_down: TensorSpec((self.hidden, self.inter))}

    def load(self, tensors, device):
        gate, up = place(tensors[self.n_gate], device, self.dtype), place(tensors[self.n_up], device, self.dtype)
        self.w_gate_up = torch.stack([gate, up], dim=1).reshape(2 * self.inter, self.hidden).contiguous()
        self.w_down = place(tensors[self.n_down], device, self.dtype)
        # where the kernels keep the activation's two constants (asked for here, outside any recording)
        # (a model on the CPU with no stand-in for the kernels only holds its weights)
        on_device = torch.device(device).type == "cuda"
        with torch.cuda.device(device) if on_device else contextlib.nullcontext():
            try:
                self.glu = kernels().glu_clamp_slot(self.limit, self.alpha) if on_device or stand_in_kernels() else None
            except KernelError:         # (every slot taken: the activation then runs as a kernel of its own on the 32-bit sums)
                self.glu = None

    def export(self):
        both = self.w_gate_up.cpu().view(self.inter, 2, self.hidden)
        return {self.n_gate: both[:, 0, :].contiguous(), self.n_up: both[:, 1, :].contiguous(), self.n_down: self.w_down.cpu()}

    def forward(self, ctx, x, h):
        k = kernels()
        T = x.shape[0]
        act = ctx.workspace("mlp.act", (T, self.inter), self.dtype)
        if self.glu is not None:
            k.gemm(x, self.w_gate_up, act, EPI_GLU_CLAMP, ctx.gemm_workspace(x, self.w_gate_up), glu=self.glu)
        else:
            sums = ctx.workspace("mlp.up", (T, 2 * self.inter), torch.float32)
            k.gemm(x, self.w_gate_up, sums, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_gate_up))
            k.act_weight(act, sums, None, self.inter, "clamped_glu", self.limit, self.alpha)
        k.gemm(act, self.w_down, h, EPI_ACCUM_F32, ctx.gemm_workspace(act, self.w_down))
        ctx.note_left(h, None)


class PlainFF(FeedForward):
    """Feed-forward without a gate(hidden_size, intermediate_size, activation): h += Wdown act(Wup x).  The up product
    leaves 32-bit sums; the activation is computed on them and rounded once to the activation type."""
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        self.activation = spec.params.get("activation", "relu2")
        if self.activation not in ACTIVATIONS or self.activation in GATED:
            raise ValueError(f"unknown activation {self.activation!r} of one projection (known: relu2)")
        leaves = {"up": "up_proj.weight", "down": "down_proj.weight", **(spec.params.get("names") or {})}
        self.n_up, self.n_down = self.name(leaves["up"]), self.name(leaves["down"])
        self.w_up = self.w_down = None

    def tensors(self):
        return {self.n_up: TensorSpec((self.inter, self.hidden)), self.n_down: TensorSpec((self.hidden, self.inter))}

    def load(self, tensors, device):
        self.w_up = place(tensors[self.n_up], device, self.dtype)
        self.w_down = place(tensors[self.n_down], device, self.dtype)

    def export(self):
        return {self.n_up: self.w_up.cpu(), self.n_down: self.w_down.cpu()}

    def forward(self, ctx, x, h):
        k = kernels()
        T = x.shape[0]
        up = ctx.workspace("mlp.up", (T, self.inter), torch.float32)
        k.gemm(x, self.w_up, up, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_up))
        act = ctx.workspace("mlp.act", (T, self.inter), self.dtype)
        k.act_weight(act, up, None, self.inter, self.activation)
        k.gemm(act, self.w_down, h, EPI_ACCUM_F32, ctx.gemm_workspace(act, self.w_down))
        ctx.note_left(h, None)


class RoutedFF(FeedForward):
    """Mixture of experts(hidden_size, intermediate_size, experts, top, activation, renormalize): each expert is a
    feed-forward without a gate; scores = softmax(Wrouter x) over all experts in 32-bit, the `top` largest are chosen,
    and the output is the sum of the chosen experts' outputs, each weighed by its score (as it is, or with
    `renormalize` divided by the chosen scores' sum).

    The experts' up matrices are laid one under the other and their down matrices side by side at load, so a step's
    experts are one up product of experts * intermediate_size columns, one pass that applies the activation and each
    column's expert weight (zero where the token did not choose the expert), and one down product: w_e Wdown_e act(.)
    = Wdown_e (w_e act(.)).  A step with a prompt portion (never one that is recorded) whose experts would each get
    `SORT_FROM_ROWS` rows or more on average lays the chosen (token, expert) pairs out expert by expert instead, and
    every expert's rows are a product of their own: top / experts of the arithmetic.  The host reads how many tokens
    each expert got (one small copy) to size those products; the down matrices are kept a second time, one by one.
    That is for experts whose matrices have `SORT_FROM_WEIGHT` elements or more: the products of smaller experts over
    a few hundred rows each leave most of the device idle, and the one product over all experts, four times the
    arithmetic at 4 of 16, is the shorter way (a prompt of 2048 tokens, 16 experts of which 4: experts of 2048 x 2048
    0.87 ms a layer in one product against 1.2 ms one by one; experts of 3584 x 4096 2.1 ms against 1.4 ms).
    Names: `router`, and `expert` with a place for the expert's number (e.g. "e{}").

    Further parameters: `activation` = "clamped_glu" (with `limit`, `alpha`): the experts have a gate projection beside
    the up projection (tensor leaf `gate`), a row of one after a row of the other in the matrix that lies under the other
    experts'; `score` = "sigmoid": each expert's score is the sigmoid of its logit by itself, the choice goes by score +
    `correction` (a tensor [experts], leaf `correction`, if `correction` is true) and the weights are the scores without
    it (`renormalize`: divided by the chosen scores' sum), times `scale`; `shared` = {kind, prefix leaf, params}: a
    feed-forward of any registered kind that every token passes beside its experts, added in."""
    graph_safe = True
    SORT_FROM_ROWS = 128
    SORT_FROM_WEIGHT = 8 << 20

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        p = spec.params
        self.hidden, self.inter = int(p["hidden_size"]), int(p["intermediate_size"])
        self.experts, self.top = int(p["experts"]), int(p["top"])
        self.renormalize = bool(p.get("renormalize", False))
        self.activation = p.get("activation", "relu2")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r} (known: {', '.join(ACTIVATIONS)})")
        self.gated = self.activation in GATED
        self.up_rows = (2 if self.gated else 1) * self.inter       # rows of an expert's part of the up matrix
        self.limit, self.alpha = float(p.get("limit", 0.0)), float(p.get("alpha", 1.702))
        if self.gated and not self.limit > 0:
            raise ValueError(f"the activation's limit must be positive, got {self.limit}")
        self.score = p.get("score", "softmax")
        if self.score not in ("softmax", "sigmoid"):
            raise ValueError(f"unknown router score {self.score!r} (known: softmax, sigmoid)")
        self.scale = float(p.get("scale", 1.0))
        self.has_correction = bool(p.get("correction", False))
        if self.score != "sigmoid" and (self.has_correction or self.scale != 1.0):
            raise ValueError("a correction of the choice and a scale of the weights go with sigmoid scores")
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"top = {self.top} of {self.experts} experts")
        leaves = {"router": "router.weight", "expert": "experts.{}", "up": "up_proj.weight", "down": "down_proj.weight", "gate": "gate_proj.weight",
                  "correction": "correction", **(p.get("names") or {})}
        self.n_router = self.name(leaves["router"])
        self.n_correction = self.name(leaves["correction"])
        self.n_up = [self.name(leaves["expert"].format(e) + "." + leaves["up"]) for e in range(self.experts)]
        self.n_gate = [self.name(leaves["expert"].format(e) + "." + leaves["gate"]) for e in range(self.experts)]
        self.n_down = [self.name(leaves["expert"].format(e) + "." + leaves["down"]) for e in range(self.experts)]
        self.w_router = self.w_up = self.w_down = self.w_down_each = self.correction = None
        shared = p.get("shared")
        self.shared = None
        if shared is not None:
            from ..config.spec import PartSpec
            self.shared = build_feed_forward(PartSpec(shared["kind"], self.name(shared["prefix"]), dict(shared["params"])), dtype)
            self.graph_safe = bool(self.shared.graph_safe)

    def tensors(self):
        t = {self.n_router: TensorSpec((self.experts, self.hidden), "normal:0.0:0.1")}
        if self.has_correction:
            t[self.n_correction] = TensorSpec((self.experts,), "normal:0.0:0.1")
        for e in range(self.experts):
            t[self.n_up[e]] = TensorSpec((self.inter, self.hidden))
            if self.gated:
                t[self.n_gate[e]] = TensorSpec((self.inter, self.hidden))
            t[self.n_down[e]] = TensorSpec((self.hidden, self.inter))
        if self.shared is not None:
            t.update(self.shared.tensors())
        return t

    def load(self, tensors, device):
        self.w_router = place(tensors[self.n_router], device, self.dtype)
        if self.has_correction:
            self.correction = place(tensors[self.n_correction], device, torch.float32)
        if self.shared is not None:
            self.shared.load(tensors, device)
        get = lambda n: place(tensors[n], device, self.dtype)
        if self.gated:      # (gate_j, up_j) row after row within each expert, the experts one under the other
            self.w_up = torch.cat([torch.stack([get(g), get(u)], dim=1).reshape(self.up_rows, self.hidden)
                                   for g, u in zip(self.n_gate, self.n_up)], dim=0).contiguous()
        else:
            self.w_up = torch.cat([get(n) for n in self.n_up], dim=0).contiguous()
        self.w_down = torch.cat([place(tensors[n], device, self.dtype) for n in self.n_down], dim=1).contiguous()
        # each expert's down matrix by itself, for the steps that run the experts one by one (not when all are chosen)
        self.w_down_each = (self.w_down.view(self.hidden, self.experts, self.inter).permute(1, 0, 2).contiguous()
                            if self.top < self.experts and self.inter * self.hidden >= self.SORT_FROM_WEIGHT else None)

    def export(self):
        up, down = self.w_up.cpu(), self.w_down.cpu()
        t = {self.n_router: self.w_router.cpu()}
        if self.has_correction:
            t[self.n_correction] = self.correction.cpu()
        for e in range(self.experts):
            mine = up[e * self.up_rows:(e + 1) * self.up_rows]
            if self.gated:
                both = mine.view(self.inter, 2, self.hidden)
                t[self.n_gate[e]], t[self.n_up[e]] = both[:, 0, :].contiguous(), both[:, 1, :].contiguous()
            else:
                t[self.n_up[e]] = mine.contiguous()
            t[self.n_down[e]] = down[:, e * self.inter:(e + 1) * self.inter].contiguous()
        if self.shared is not None:
            t.update(self.shared.export())
        return t

    def step_weight_bytes(self, seen):
        # a single token reads the router and the experts it chose
        if self.w_down_each is not None:
            seen.add(self.w_down_each.data_ptr())          # (the second copy of the down matrices: a step reads one of the two)
        total = super().step_weight_bytes(seen)
        experts = (self.w_up.numel() + self.w_down.numel()) * self.w_up.element_size()
        shared = self.shared.step_weight_bytes(seen) if self.shared is not None else 0
        return total - experts + experts * self.top // self.experts + shared

    def forward(self, ctx, x, h):
        k = kernels()
        T, N = x.shape[0], self.experts * self.inter
        logits = ctx.workspace("moe.logits", (T, self.experts), torch.float32)
        k.gemm(x, self.w_router, logits, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_router))
        weights = ctx.workspace("moe.weights", (T, self.experts), torch.float32)
        if self.score == "sigmoid":
            k.route_topk(logits, weights, self.top, self.renormalize, "sigmoid", self.correction, self.scale)
        else:
            k.route_topk(logits, weights, self.top, self.renormalize)
        if self.shared is not None:         # (reads x, adds into h; the experts' buffers are its own until it is done)
            self.shared.forward(ctx, x, h)
        if (self.w_down_each is not None and ctx.longest > 1 and T * self.top >= self.SORT_FROM_ROWS * self.experts
                and self.inter * self.hidden >= self.SORT_FROM_WEIGHT):
            return self._forward_sorted(ctx, x, h, weights)
        up = ctx.workspace("mlp.up", (T, self.experts * self.up_rows), torch.float32)
        k.gemm(x, self.w_up, up, EPI_STORE_F32, ctx.gemm_workspace(x, self.w_up))
        act = ctx.workspace("mlp.act", (T, N), self.dtype)
        k.act_weight(act, up, weights, self.inter, self.activation, self.limit, self.alpha)
        k.gemm(act, self.w_down, h, EPI_ACCUM_F32, ctx.gemm_workspace(act, self.w_down))
        ctx.note_left(h, None)


    def _forward_sorted(self, ctx, x, h, weights):
        k = kernels()
        T, E, F, D = x.shape[0], self.experts, self.inter, self.hidden
        rows = T * self.top
        counts = ctx.workspace("moe.counts", (E,), torch.int32)
        k.route_counts(weights, counts)
        n_of = counts.cpu().tolist()                 # (the step waits here: the experts' products are sized by these)
        total = sum(n_of)                            # (a chosen expert whose score is exactly zero has no row: it adds nothing)
        assert total <= rows
        row_token = ctx.workspace("moe.row_token", (rows,), torch.int32)
        row_weight = ctx.workspace("moe.row_weight", (rows, 1), torch.float32)
        row_of = ctx.workspace("moe.row_of", (T, E), torch.int32)
        k.route_rows(weights, counts, row_token, row_weight, row_of)
        if total == 0:
            return ctx.note_left(h, None)
        xs = ctx.workspace("moe.x", (rows, D), self.dtype)[:total]
        k.gather_rows(xs, x, row_token[:total])
        U = self.up_rows
        up = ctx.workspace("mlp.up", (rows, U), torch.float32)[:total]
        at = 0
        for e, n in enumerate(n_of):
            if n:
                w = self.w_up[e * U:(e + 1) * U]
                k.gemm(xs[at:at + n], w, up[at:at + n], EPI_STORE_F32, ctx.gemm_workspace(xs[at:at + n], w))
                at += n
        act = ctx.workspace("mlp.act", (rows, F), self.dtype)[:total]
        k.act_weight(act, up, row_weight[:total], F, self.activation, self.limit, self.alpha)
        ys = ctx.workspace("moe.y", (rows, D), torch.float32)[:total]
        at = 0
        for e, n in enumerate(n_of):
            if n:
                w = self.w_down_each[e]
                k.gemm(act[at:at + n], w, ys[at:at + n], EPI_STORE_F32, ctx.gemm_workspace(act[at:at + n], w))
                at += n
        k.combine_rows(h, ys, row_of)
        ctx.note_left(h, None)


register_feed_forward("clamped_glu", ClampedGLU)
register_feed_forward("plain_ff", PlainFF)
register_feed_forward("routed_ff", RoutedFF)

"""Norms.  RMSNorm(size, eps): y = x / sqrt(mean(x^2) + eps) * weight, computed in 32-bit,
the weight multiplying directly.  Reference: rms_norm_batch
(shaders/ops.metal:970-1003), used at src/arch/llama.rs:152,164,135."""
from __future__ import annotations

import torch

from ..kernels import NormedRows, kernels
from .base import Norm, TensorSpec, place, register_norm


class RMSNorm(Norm):
    """`tensor`: the leaf of the weight's name ("weight"); "" when the prefix itself is the name."""
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        leaf = spec.params.get("tensor", "weight")
        self.weight_name = self.name(leaf) if leaf else self.prefix
        self.weight = None

    def tensors(self):
        return {self.weight_name: TensorSpec((self.size,), "norm")}

    def load(self, tensors, device):
        # The reference wants norm weights in 32-bit (ops.metal:972); whatever the
        # file stores, the kernel multiplies by a float32 weight.
        self.weight = place(tensors[self.weight_name], device, torch.float32)

    def export(self):
        return {self.weight_name: self.weight.cpu()}

    def forward(self, ctx, h, out, rows=None):
        kernels().rmsnorm(out, h, self.weight, self.eps, rows)

    def forward_clearing(self, ctx, h, out, zero):
        kernels().group_rmsnorm(out, h, self.weight, self.eps, 1, zero=zero)       # (one group: this norm; clears on the way)

    def add_normed(self, ctx, y, h):
        kernels().rmsnorm_sum(h, [(y, None, self.weight)], 1.0, self.eps)

    def deferred_weight(self):
        return self.weight

    def deferred_eps(self):
        return self.eps

    def deferred(self, ctx, h):
        left = ctx.left_for(h)
        if left is None or left.weight is not self.weight or h.shape[1] != self.size or left.y.shape != h.shape:
            return None         # nothing was left, or it was prepared for another norm
        if left.whole:          # finished by the product that added into the stream last
            return left.y if left.eps == self.eps else None
        return NormedRows(left.y, left.sumsq, self.eps)


register_norm("rmsnorm", RMSNorm)


class GroupRMSNorm(Norm):
    """RMS norm in groups(size, eps, groups): the row is cut into `groups` equal consecutive parts, each part p becomes
    p / sqrt(mean(p^2) + eps), and the whole is multiplied by the weight; 32-bit throughout.  groups = 1 is RMSNorm.
    It also reads a stream kept in several copies, combined with given weights on the way (`forward_streams`).
    `tensor`: the leaf of the weight's name ("weight"); "" when the prefix itself is the name."""
    graph_safe = True
    FUSE_MIX_FROM_ROWS = 128

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.groups = int(spec.params.get("groups", 1))
        if self.groups < 1 or self.size % self.groups:
            raise ValueError(f"a row of {self.size} does not fall into {self.groups} equal groups")
        leaf = spec.params.get("tensor", "weight")
        self.weight_name = self.name(leaf) if leaf else self.prefix
        self.weight = None

    def tensors(self):
        return {self.weight_name: TensorSpec((self.size,), "norm")}

    def load(self, tensors, device):
        self.weight = place(tensors[self.weight_name], device, torch.float32)

    def export(self):
        return {self.weight_name: self.weight.cpu()}

    def forward(self, ctx, h, out, rows=None):
        kernels().group_rmsnorm(out, h, self.weight, self.eps, self.groups, rows)

    def forward_streams(self, ctx, hs, w_in, out, rows=None, zero=None):
        # A mix of these streams that is still to be done runs in the norm's launch, when the norm reads every row
        # and there are rows enough to fill the device with one block a row (the mix alone spreads a row over blocks).
        mix = ctx.take_streams_mix(hs) if rows is None and hs.shape[1] >= self.FUSE_MIX_FROM_ROWS else None
        if mix is None:
            ctx.flush_streams()
        kernels().group_rmsnorm(out, hs, self.weight, self.eps, self.groups, rows, w_in=w_in, zero=zero, mix=mix)
        return True


register_norm("group_rmsnorm", GroupRMSNorm)


class DynamicTanh(Norm):
    """Dynamic tanh(size): y = tanh(alpha x) weight + bias, with one scalar alpha for the whole row, a weight and a bias
    per feature; nothing is summed over the row (no mean, no variance, no eps).  32-bit throughout, one rounding on the
    way out.  Tensors: the weight under the prefix itself, the bias under `<prefix>.b`, the scalar under
    `<prefix>.alpha` (`names` gives other leaves).  Two such norms of the same rows run in one launch that reads the
    rows once (`forward_with`)."""
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.size = int(spec.params["size"])
        leaves = {"weight": "", "bias": "b", "alpha": "alpha", **(spec.params.get("names") or {})}
        self.names = {key: (self.name(leaf) if leaf else self.prefix) for key, leaf in leaves.items()}
        self.weight = self.bias = self.alpha = None

    def tensors(self):
        n = self.names
        return {n["weight"]: TensorSpec((self.size,), "norm"), n["bias"]: TensorSpec((self.size,), "normal:0.0:0.1"),
                n["alpha"]: TensorSpec((), "normal:0.6:0.1")}

    def load(self, tensors, device):
        get = lambda key: place(tensors[self.names[key]], device, torch.float32)
        self.weight, self.bias = get("weight"), get("bias")
        self.alpha = get("alpha").reshape(1)            # stays on the device: the kernel reads it there

    def export(self):
        n = self.names
        return {n["weight"]: self.weight.cpu(), n["bias"]: self.bias.cpu(), n["alpha"]: self.alpha.cpu().reshape(())}

    def forward(self, ctx, h, out, rows=None):
        kernels().dyt(out, h, self.weight, self.bias, self.alpha, rows)

    def forward_with(self, ctx, h, out, other, other_out) -> bool:
        """out = this norm of every row of h and other_out = `other`'s, in one launch; False when `other` is of
        another kind (the caller then runs the two one after the other)."""
        if not isinstance(other, DynamicTanh) or other.size != self.size:
            return False
        kernels().dyt(out, h, self.weight, self.bias, self.alpha, None, second=(other_out, other.weight, other.bias, other.alpha))
        return True


register_norm("dyt", DynamicTanh)


class LayerNorm(Norm):
    """Layer norm(size, eps) with weight and bias: y = (x - mean) / sqrt(var + eps) * weight + bias, var the mean of the
    squared deviations from the mean.  32-bit throughout, one rounding on the way out.  Tensors: the weight under the
    prefix itself, the bias under `<prefix>.b` (`names` gives other leaves)."""
    graph_safe = True

    def __init__(self, spec, dtype):
        super().__init__(spec, dtype)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        leaves = {"weight": "", "bias": "b", **(spec.params.get("names") or {})}
        self.names = {key: (self.name(leaf) if leaf else self.prefix) for key, leaf in leaves.items()}
        self.weight = self.bias = None

    def tensors(self):
        return {self.names["weight"]: TensorSpec((self.size,), "norm"), self.names["bias"]: TensorSpec((self.size,), "normal:0.0:0.1")}

    def load(self, tensors, device):
        self.weight = place(tensors[self.names["weight"]], device, torch.float32)
        self.bias = place(tensors[self.names["bias"]], device, torch.float32)

    def export(self):
        return {self.names["weight"]: self.weight.cpu(), self.names["bias"]: self.bias.cpu()}

    def forward(self, ctx, h, out, rows=None):
        kernels().layernorm(out, h, self.weight, self.bias, self.eps, rows)


register_norm("layernorm", LayerNorm)

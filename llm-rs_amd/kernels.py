"""The kernel interface: every device operation of the engine goes through the
object `kernels()` returns.  It is the gfx950 library (csrc/hip) or nothing:
when that library cannot be built or loaded, or there is no GPU, the first use
raises.  `use_kernels()` lets a test put another object with the same methods in
its place; the package itself never does.

Op set of the reference's `Backend` trait (src/backend/mod.rs:15-89), fused:
embed, rms_norm, matmul (+ residual add / SwiGLU epilogues for add/silu/mul),
rope + scatter_kv, attention, gather (folded into rms_norm's row list), argmax.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
import sys
from ctypes import c_char_p, c_float, c_int, c_size_t, c_void_p
from typing import Dict, List, NamedTuple, Optional

import torch

EPI_STORE, EPI_STORE_F32, EPI_ACCUM_F32, EPI_SWIGLU = 0, 1, 2, 3
EPI_GLU_CLAMP = 5       # and what `glu_clamp_slot` gave is added to it (4 is the kernel library's own: the q/k/v epilogue of `qkv_rope_cache`)
_EPI_NAMES = {EPI_STORE: "store", EPI_STORE_F32: "store32", EPI_ACCUM_F32: "add32", EPI_SWIGLU: "swiglu", EPI_GLU_CLAMP: "clamped glu"}
_EPI_GATED = (EPI_SWIGLU, EPI_GLU_CLAMP)

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


# MI355X, published: HBM3E 8 TB/s; dense matrix cores 2.5 PFLOP/s in bfloat16, 157.3 TFLOP/s in float32
PEAK_HBM_BYTES = 8.0e12
PEAK_FLOPS = {torch.bfloat16: 2.5e15, torch.float32: 157.3e12}


class KernelError(RuntimeError):
    pass


class NormedRows:
    """Rows whose norm is left to the product that takes them (steps of a few tokens; no norm kernel runs).
    `y` [rows, K] holds the stream's rows times the norm's weight, rounded once to the activation type, and
    `sumsq` [rows, parts] the sums of squares of each 16 consecutive features of the stream's rows: both left
    by the product that added into the stream last.  The product multiplies each of its 32-bit sums by the row's
    1 / sqrt(sum(sumsq) / K + eps): x W^T with x = h inv weight equals inv (h weight) W^T."""

    def __init__(self, y: torch.Tensor, sumsq: torch.Tensor, eps: float):
        self.y, self.sumsq, self.eps = y, sumsq, float(eps)
        self.shape, self.dtype = y.shape, y.dtype


class NextNorm:
    """What a product that adds into the stream leaves for the norm that follows, see `NormedRows`:
    `y` and `sumsq` to fill, `weight` the following norm's.  With `eps` (and no `sumsq`) the product finishes the
    norm itself: `y` becomes the normed rows, for any product to take as they are (`gemm_norms_whole`: steps of
    17 tokens or more whose product is split over blocks, where the kernel that adds the parts up sees whole rows)."""

    def __init__(self, y: torch.Tensor, sumsq: Optional[torch.Tensor], weight: torch.Tensor, eps: float = 0.0):
        self.y, self.sumsq, self.weight, self.eps = y, sumsq, weight, float(eps)

    @property
    def whole(self) -> bool:
        return self.eps > 0.0


class KernelTimes:
    """Per-kernel device time with the bytes each call has to move and the operations it has to
    do, as the reference keeps when LLM_PERF is set (src/backend/metal/mod.rs:321-400): a pair of
    events around every call, read when the table is asked for."""

    def __init__(self):
        self.calls: List[tuple] = []       # (label, bytes, flops, peak flops, start event, end event)

    def add(self, label, nbytes, flops, peak, start, end):
        self.calls.append((label, nbytes, flops, peak, start, end))

    def rows(self) -> List[dict]:
        """One row per label, most device time first; clears what was recorded."""
        torch.cuda.synchronize()
        acc: Dict[str, dict] = {}
        for label, nbytes, flops, peak, start, end in self.calls:
            r = acc.setdefault(label, {"kernel": label, "calls": 0, "seconds": 0.0, "bytes": 0, "flops": 0, "peak_flops": peak})
            r["calls"] += 1
            r["seconds"] += start.elapsed_time(end) * 1e-3
            r["bytes"] += nbytes
            r["flops"] += flops
        self.calls = []
        rows = sorted(acc.values(), key=lambda r: -r["seconds"])
        for r in rows:
            t = max(r["seconds"], 1e-12)
            r["gb_per_s"] = r["bytes"] / t / 1e9
            r["hbm_frac"] = r["bytes"] / t / PEAK_HBM_BYTES
            r["tflops"] = r["flops"] / t / 1e12
            r["flops_frac"] = r["flops"] / t / r["peak_flops"] if r["peak_flops"] else 0.0
        return rows

    def dump(self, file=None) -> List[dict]:
        file = file or sys.stderr
        rows = self.rows()
        if not rows:
            return rows
        total = sum(r["seconds"] for r in rows)
        print(f"  {'kernel':<34} {'calls':>6} {'GPU time':>10} {'% total':>8}  {'GB/s (% of 8 TB/s)':>20}  {'TFLOP/s (% of peak)':>20}", file=file)
        print("  " + "-" * 106, file=file)
        for r in rows:
            t = f"{r['seconds'] * 1e3:.2f}ms" if r["seconds"] >= 1e-3 else f"{r['seconds'] * 1e6:.0f}us"
            fl = f"{r['tflops']:.1f} ({r['flops_frac'] * 100:.1f}%)" if r["flops"] else "-"
            print(f"  {r['kernel']:<34} {r['calls']:>6} {t:>10} {r['seconds'] / total * 100:>7.1f}%  "
                  f"{r['gb_per_s']:>10.0f} ({r['hbm_frac'] * 100:>4.1f}%)  {fl:>20}", file=file)
        all_bytes = sum(r["bytes"] for r in rows)
        print("  " + "-" * 106, file=file)
        print(f"  {'TOTAL':<34} {'':>6} {total * 1e3:>8.2f}ms {'100.0%':>8}  {all_bytes / total / 1e9:>10.0f} ({all_bytes / total / PEAK_HBM_BYTES * 100:>4.1f}%)",
              file=file)
        return rows


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}") from None


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


class NormPlan(NamedTuple):
    """How a product that adds into the stream serves the norm that follows it (`Kernels.norm_left_by_product`)."""
    whole: bool          # True: the product finishes the norm itself (a `NextNorm` with eps, and the product's workspace)
    parts: int           # else: partial sums of squares it leaves per row, the second dimension of `NextNorm.sumsq`


class Kernels:
    """What the engine asks of its device operations beyond the operations themselves: how much room a call needs and
    which of the optional hand-overs between kernels a call can take.  An implementation answers for itself; the
    answers here are those of one that splits nothing and hands nothing over, so that parts never have to probe the
    object they were given."""

    allow_mfma = False
    times: Optional[KernelTimes] = None

    def gemm_workspace_floats(self, M: int, N: int, K: int) -> int:
        """Room (floats) that lets the product of M rows with an [N, K] weight split K over blocks; 0: none needed."""
        return 0

    def product_norms_its_rows(self, M: int, N: int, K: int, dtype: torch.dtype) -> bool:
        """Whether the product of M rows with an [N, K] weight takes `NormedRows` (rows still to be scaled by
        their norm) in place of normed rows."""
        return False

    def norm_left_by_product(self, M: int, N: int, K: int, dtype: torch.dtype) -> Optional[NormPlan]:
        """What the product of M rows with an [N, K] weight, adding into the stream, can leave for the norm that
        reads the stream next (`NextNorm`), or None: then a norm kernel runs."""
        return None

    def attention_scratch_floats(self, n_entries: int, n_heads: int, head_dim: int, max_seq_len: int,
                                 n_kv_heads: Optional[int] = None, n_single: int = 0) -> int:
        """Room (floats) for the partial results of single-token entries whose keys are shared out over waves."""
        return 0

    def attention_split_chunk(self, n_single: int, n_kv_heads: int, head_dim: int, max_seq_len: int, single_keys: int = 0) -> int:
        """Keys per wave that a call with these figures splits its single-token entries by (0: it does not split):
        what a caller that records steps has to key its recordings by."""
        return 0


class HipKernels(Kernels):
    """Launches on the current torch stream of the tensors' device."""

    def __init__(self):
        from .csrc.build import load_hip
        if not torch.cuda.is_available():
            raise KernelError("no GPU: the engine's kernels are gfx950 HIP kernels and there is no other path")
        self.lib = lib = load_hip()
        lib.llmrs_hip_error.restype = c_char_p
        V, I, F = c_void_p, c_int, c_float
        sigs = {
            "llmrs_embed_rows": [V, I, V, V, V, I, I, I, F],
            "llmrs_embed_rows_add": [V, I, V, V, V, I, I, I, F],
            "llmrs_dyt": [V, I, V, V, V, V, V, V, I, I, V, V, V, V],
            "llmrs_conv_state_update": [V, V, I, V, ctypes.c_long, V, V, I, I, I],
            "llmrs_sigmoid_gate": [V, I, V, I, V, I, I, I, I],
            "llmrs_latent_finish": [V, I, V, I, V, I, I, I, I, V, F, V, V, V, I, I, I, V, I, V, V, F],
            "llmrs_layernorm": [V, I, V, V, V, V, V, I, I, F],
            "llmrs_exp_gates": [V, V, V, I, V, V, F, V, ctypes.c_long, V, V, I, I, I, V, V, V, I],
            "llmrs_qkv_whole": [V, V, I, I, I, I, I, V, V, F, V, I, V, V, I],
            "llmrs_head_product": [V, I, V, I, V, V, I, I, I, I, I, I, V, I],
            "llmrs_fill_normal": [V, I, V, c_size_t, ctypes.c_uint64, ctypes.c_uint64, F, F],
            "llmrs_cast": [V, V, I, V, I, c_size_t],
            "llmrs_scale_softcap_rows": [V, V, I, I, I, F, F],
            "llmrs_rmsnorm": [V, I, V, V, V, V, I, I, F],
            "llmrs_gemm": [V, I, V, I, V, V, I, I, I, I, I, V, c_size_t, I, V, I, F, V, V, I, V, F],
            "llmrs_glu_clamp_slot": [V, F, F],
            "llmrs_gemm_defers_norm": [I, I, I],
            "llmrs_gemm_norms_whole": [I, I, I],
            "llmrs_gemm_next_parts": [I, I, I],
            "llmrs_rope_kv_write": [V, I, V, I, V, V, V, I, I, V, V, I, I, I, I, I, I, I],
            "llmrs_attention": [V, I, V, I, V, I, V, V, V, I, V, V, V, V, I, I, I, I, I, I, I, I, F, V, c_size_t, I, I, ctypes.c_long, I],
            "llmrs_qkv_rope_cache": [V, I, V, I, V, V, I, I, I, V, V, V, I, V, V, I, I, I, I, I, I, V, c_size_t, I, V, I, F],
            "llmrs_argmax_rows": [V, V, I, I, I, V, V, c_size_t],
            "llmrs_sample_rows": [V, V, I, I, I, V, V],
            "llmrs_place_ids": [V, V, I, V, V, V, I, I, I],
            "llmrs_attention_ext": [V, I, V, I, V, I, V, V, V, I, V, V, V, V, I, I, I, I, I, I, I, I, F, V, c_size_t, I, I, ctypes.c_long, I, I, V, V, F, I, V, V, I, I],
            "llmrs_group_rmsnorm": [V, I, V, V, ctypes.c_long, I, V, V, V, I, I, I, F, V, V, V, V, V],
            "llmrs_streams_mix": [V, V, ctypes.c_long, I, V, V, V, ctypes.c_long],
            "llmrs_streams_copy_first": [V, V, ctypes.c_long, I, ctypes.c_long],
            "llmrs_qkv_finish": [V, I, V, I, V, V, I, V, V, V, I, I, I, I, I, I, I, I, F, V, V, I, V, V, F, V, I, V, ctypes.c_long, V, V, V, I],
            "llmrs_linear_scan": [V, V, I, V, I, V, I, V, I, V, V, I, V, ctypes.c_long, V, V, I, I, I, I, I, I, V, I, V, V, I, I],
            "llmrs_silu_columns": [V, V, I, I, I, I],
            "llmrs_delta_prepare": [V, V, I, V, I, V, I, V, I, V, V, I, I, I, I, F],
            "llmrs_gated_rmsnorm": [V, I, V, I, V, I, V, I, I, I, I, F, V, I, I, V, I, F, F],
            "llmrs_rmsnorm_sum": [V, V, V, V, V, V, V, V, I, I, F, F],
            "llmrs_route_topk": [V, V, I, V, I, I, I, I, I, I, V, F],
            "llmrs_act_weight": [V, I, V, I, V, I, I, I, I, I, V, I, F, F],
            "llmrs_add_bias_rows": [V, V, I, V, I, I],
            "llmrs_route_counts": [V, V, I, I, I, V],
            "llmrs_route_rows": [V, V, I, I, I, V, V, V, V],
            "llmrs_gather_rows": [V, I, V, I, V, I, V, I, I],
            "llmrs_combine_rows": [V, V, I, V, I, V, I, I, I],
            "llmrs_mingru_scan": [V, I, V, I, V, V, V, ctypes.c_long, V, V, I, I, V, I, I, V],
            "llmrs_causal_conv_silu": [V, I, V, I, V, V, V, ctypes.c_long, V, V, V, I, I, I, I, V, I],
            "llmrs_selective_scan": [V, I, V, I, V, I, I, I, V, I, V, V, V, V, I, V, ctypes.c_long, V, V, V, I, I, I, I, V, I, I, V],
        }
        for name, args in sigs.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = I
        buf = ctypes.create_string_buffer(64)
        lib.llmrs_device_arch.argtypes = [c_char_p, I]
        lib.llmrs_device_arch.restype = I
        self.compute_units = lib.llmrs_device_arch(buf, 64)
        self.arch = buf.value.decode()
        if not self.arch.startswith("gfx950"):
            raise KernelError(f"the kernel library is built for gfx950, the device is {self.arch!r}")
        self.allow_mfma = True  # tests switch the matrix-core kernels off to compare paths
        # LLM_PERF in the environment (the reference's switch): every call is timed on the device and
        # steps are not recorded into graphs, so that each kernel can be seen by itself
        self.times: Optional[KernelTimes] = KernelTimes() if os.environ.get("LLM_PERF") else None
        lib.llmrs_attention_scratch_floats.restype = ctypes.c_long
        lib.llmrs_scan_places.argtypes = [ctypes.c_long, ctypes.c_long]
        lib.llmrs_scan_places.restype = ctypes.c_long
        lib.llmrs_scan_chunk.argtypes = []
        lib.llmrs_scan_chunk.restype = I
        self.scan_chunk = lib.llmrs_scan_chunk()
        lib.llmrs_scan_set_chunk.argtypes = [I]
        lib.llmrs_scan_set_chunk.restype = I
        lib.llmrs_attention_scratch_floats.argtypes = [I, I, I, I, I, I]
        lib.llmrs_attention_split_chunk.restype = I
        lib.llmrs_attention_split_chunk.argtypes = [ctypes.c_long, I, I, I, ctypes.c_long]
        lib.llmrs_gemm_workspace_floats.restype = ctypes.c_long
        lib.llmrs_gemm_workspace_floats.argtypes = [I, I, I]

    def gemm_workspace_floats(self, M: int, N: int, K: int) -> int:
        """Room that lets a product with too few blocks split K over blocks (the kernels' own rule)."""
        return int(self.lib.llmrs_gemm_workspace_floats(int(M), int(N), int(K)))

    def product_norms_its_rows(self, M: int, N: int, K: int, dtype: torch.dtype) -> bool:
        return dtype == torch.bfloat16 and self.gemm_defers_norm(M, N, K)

    def norm_left_by_product(self, M: int, N: int, K: int, dtype: torch.dtype) -> Optional[NormPlan]:
        if dtype != torch.bfloat16:
            return None
        # up to a few rows: partial sums of squares, for the next product to finish (the kernels keep at most 1024
        # of them a row); more rows: a product that is split over blocks finishes the norm where its parts are added up
        if N < 16384 and self.gemm_defers_norm(M, N, K):
            return NormPlan(False, self.gemm_next_parts(M, N, K))
        if self.gemm_norms_whole(M, N, K):
            return NormPlan(True, 0)
        return None

    def gemm_defers_norm(self, M: int, N: int, K: int) -> bool:
        """Whether the bfloat16 product of M rows with an [N, K] weight takes `NormedRows` as its rows and, adding
        into the stream, leaves a `NextNorm` (that: for fewer than 16384 features)."""
        return self.allow_mfma and bool(self.lib.llmrs_gemm_defers_norm(int(M), int(N), int(K)))

    def gemm_next_parts(self, M: int, N: int, K: int) -> int:
        """Partial sums of squares per row that a product leaving a `NextNorm` writes (one per 16 features, for some
        shapes per 8): the second dimension of `NextNorm.sumsq`."""
        return int(self.lib.llmrs_gemm_next_parts(int(M), int(N), int(K)))

    def gemm_norms_whole(self, M: int, N: int, K: int) -> bool:
        """Whether the bfloat16 product of M rows with an [N, K] weight, adding into the stream with the workspace
        `gemm_workspace_floats` asks for, can finish the norm that follows (a `NextNorm` with eps)."""
        return self.allow_mfma and bool(self.lib.llmrs_gemm_norms_whole(int(M), int(N), int(K)))

    def attention_scratch_floats(self, n_entries: int, n_heads: int, head_dim: int, max_seq_len: int,
                                 n_kv_heads: Optional[int] = None, n_single: int = 0) -> int:
        """Room the split of single-token entries needs for its partial results (the kernels' own rule: the key
        ranges get shorter when there are few such entries)."""
        return int(self.lib.llmrs_attention_scratch_floats(int(n_entries), int(n_single), int(n_heads),
                                                            int(n_kv_heads or n_heads), int(head_dim), int(max_seq_len)))

    def _check(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self.lib.llmrs_hip_error().decode())

    def _run(self, label: str, nbytes: int, flops: int, dtype, fn, *args) -> None:
        """Calls the library; with timing on, between two events, noting what the call has to move and to compute."""
        if self.times is None:
            return self._check(fn(*args))
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        self._check(fn(*args))
        end.record()
        self.times.add(label, int(nbytes), int(flops), PEAK_FLOPS.get(dtype, 0.0), start, end)

    @staticmethod
    def _stream() -> int:
        return torch.cuda.current_stream().cuda_stream

    # out[t, :] = table[tokens[t], :] * scale as float32
    # (add: out[t, :] += the same, for a stream that is shown its tokens' embeddings again)
    def embed_rows(self, out: torch.Tensor, table: torch.Tensor, tokens: torch.Tensor, scale: float = 1.0, add: bool = False) -> None:
        assert out.dtype == torch.float32 and tokens.dtype == torch.int32 and table.is_contiguous() and out.is_contiguous()
        assert out.shape[0] == tokens.shape[0] and out.shape[1] == table.shape[1]
        self._run("embed add" if add else "embed", out.numel() * ((8 if add else 4) + table.element_size()), out.numel() if add else 0, None,
                  self.lib.llmrs_embed_rows_add if add else self.lib.llmrs_embed_rows, self._stream(), _code(table.dtype), _p(out), _p(table), _p(tokens),
                  tokens.shape[0], table.shape[1], table.shape[0], float(scale))

    # out.flat[i] = mean + std * normal(seed, first + i): the same bits as the host library makes
    def fill_normal(self, out: torch.Tensor, seed: int, mean: float, std: float, first: int = 0) -> None:
        assert out.is_contiguous()
        self._check(self.lib.llmrs_fill_normal(self._stream(), _code(out.dtype), _p(out), out.numel(), seed & (2**64 - 1),
                                               int(first), float(mean), float(std)))

    # dst = src in dst's dtype (float32, bfloat16; src may be float16 too), both on the device
    def cast(self, dst: torch.Tensor, src: torch.Tensor) -> None:
        codes = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
        assert dst.is_contiguous() and src.is_contiguous() and dst.numel() == src.numel()
        if dst.dtype not in (torch.float32, torch.bfloat16) or src.dtype not in codes:
            raise KernelError(f"no cast from {src.dtype} to {dst.dtype}")
        self._check(self.lib.llmrs_cast(self._stream(), _p(dst), codes[dst.dtype], _p(src), codes[src.dtype], src.numel()))

    # logits <- logits * scale, then cap * tanh(logits / cap) if cap > 0, in place
    def scale_softcap_rows(self, logits: torch.Tensor, scale: float, cap: float) -> None:
        assert logits.dtype == torch.float32 and logits.stride(1) == 1
        self._check(self.lib.llmrs_scale_softcap_rows(self._stream(), _p(logits), logits.stride(0), logits.shape[0],
                                                      logits.shape[1], float(scale), float(cap)))

    # out[i, :] = rmsnorm(x[rows[i] or i, :]) * weight
    def rmsnorm(self, out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float,
                rows: Optional[torch.Tensor] = None) -> None:
        assert x.dtype == torch.float32 and weight.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous()
        n = out.shape[0]
        assert out.shape[1] == x.shape[1] == weight.shape[0]
        assert (rows is None and n == x.shape[0]) or (rows is not None and rows.dtype == torch.int32 and rows.shape[0] == n)
        self._run(f"rmsnorm {n}x{x.shape[1]}", n * x.shape[1] * (4 + out.element_size()) + x.shape[1] * 4, 5 * n * x.shape[1], None,
                  self.lib.llmrs_rmsnorm, self._stream(), _code(out.dtype), _p(out), _p(x), _p(weight), _p(rows),
                  n, x.shape[1], eps)

    def dyt(self, out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, alpha: torch.Tensor,
            rows: Optional[torch.Tensor] = None, second=None) -> None:
        """out[i, :] = tanh(alpha * x[rows[i] or i, :]) * weight + bias; alpha is one number on the device.
        second = (out2, weight2, bias2, alpha2): a second such norm of the same rows (every row), in the same pass."""
        n, D = out.shape
        assert x.dtype == weight.dtype == bias.dtype == alpha.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous()
        assert x.shape[1] == D == weight.numel() == bias.numel() and alpha.numel() == 1
        assert (rows is None and n == x.shape[0]) or (rows is not None and rows.dtype == torch.int32 and rows.shape[0] == n)
        out2 = w2 = b2 = a2 = None
        if second is not None:
            out2, w2, b2, a2 = second
            assert rows is None and out2.shape == out.shape and out2.dtype == out.dtype and out2.is_contiguous()
            assert w2.dtype == b2.dtype == a2.dtype == torch.float32 and w2.numel() == b2.numel() == D and a2.numel() == 1
        outs = 1 if second is None else 2
        self._run(f"dyt {n}x{D}" + (" twice" if second is not None else ""), n * D * (4 + outs * out.element_size()), 12 * outs * n * D, None,
                  self.lib.llmrs_dyt, self._stream(), _code(out.dtype), _p(out), _p(x), _p(weight), _p(bias), _p(alpha), _p(rows),
                  n, D, _p(out2), _p(w2), _p(b2), _p(a2))

    def layernorm(self, out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float,
                  rows: Optional[torch.Tensor] = None) -> None:
        """out[i, :] = (x[r] - mean) / sqrt(var + eps) * weight + bias with r = rows[i] or i, var the mean of the squared
        deviations; x, weight, bias float32."""
        n, D = out.shape
        assert x.dtype == weight.dtype == bias.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous()
        assert x.shape[1] == D == weight.numel() == bias.numel() and weight.is_contiguous() and bias.is_contiguous()
        assert (rows is None and n == x.shape[0]) or (rows is not None and rows.dtype == torch.int32 and rows.shape[0] == n)
        self._run(f"layernorm {n}x{D}", n * D * (4 + out.element_size()) + D * 8, 8 * n * D, None, self.lib.llmrs_layernorm,
                  self._stream(), _code(out.dtype), _p(out), _p(x), _p(weight), _p(bias), _p(rows), n, D, float(eps))

    def conv_state_update(self, sums: torch.Tensor, state: torch.Tensor, q_starts, slots, channels: int, taps: int) -> None:
        """state [slots, >= (taps - 1) * channels] float32 becomes each request's last taps - 1 rows of (old state, this
        step's rows of sums [T, channels]): what a causal convolution over `taps` taps reads before an entry's first token."""
        assert sums.dtype == state.dtype == torch.float32 and sums.stride(1) == 1 and sums.shape[1] == channels
        assert state.stride(-1) == 1 and state.shape[1] >= (taps - 1) * channels and q_starts.dtype == slots.dtype == torch.int32
        self._run("conv_state", 2 * slots.numel() * (taps - 1) * channels * 4, 0, None, self.lib.llmrs_conv_state_update,
                  self._stream(), _p(sums), sums.stride(0), _p(state), state.stride(0), _p(q_starts), _p(slots), slots.numel(), channels, taps)

    def sigmoid_gate(self, o: torch.Tensor, gate: torch.Tensor, per: int) -> None:
        """o[t, j] *= sigmoid(gate[t, j // per]) in place; gate float32 (a product's sums), the sigmoid and the product 32-bit."""
        T, N = o.shape
        assert gate.dtype == torch.float32 and o.stride(1) == 1 and gate.stride(1) == 1 and gate.shape[0] == T
        assert per >= 1 and N % per == 0 and gate.shape[1] == N // per
        self._run(f"sigmoid_gate {T}x{N}", T * N * 2 * o.element_size() + T * (N // per) * 4, 6 * T * N, None, self.lib.llmrs_sigmoid_gate,
                  self._stream(), _code(o.dtype), _p(o), o.stride(0), _p(gate), gate.stride(0), T, N, per)

    def latent_finish(self, sums: torch.Tensor, q: torch.Tensor, q_size: int, rank: int, weight: torch.Tensor, eps: float, slot_map,
                      k_cache: torch.Tensor, v_cache: torch.Tensor, page_size: int, num_pages: int, write: bool,
                      q_weight: Optional[torch.Tensor] = None, rotated=None) -> None:
        """sums [T, q | c | rotated part | ...] float32 -> q [T, q_size] in the activation type (as it is, or with `q_weight`
        [q_size] RMS-normed over its width and multiplied by it), and c = rmsnorm(sums_c) * weight into the cache's pages
        twice, as a row of `k_cache` [page][slot][width] and as a column of `v_cache` [page][width][slot].
        rotated = (columns, positions, inv_freq [columns / 2], gain): that many columns behind c are a key part that all
        heads share; its features (2i, 2i + 1) are turned by positions[t] * inv_freq[i], cosine and sine times gain, and
        written behind c (width = rank + columns; else width = rank)."""
        T = sums.shape[0]
        rot, positions, inv_freq, gain = rotated if rotated is not None else (0, None, None, 1.0)
        width = rank + rot
        assert sums.dtype == weight.dtype == torch.float32 and sums.stride(1) == 1 and sums.shape[1] >= q_size + width
        assert q.shape == (T, q_size) and q.stride(1) == 1 and weight.numel() == rank
        assert q_weight is None or (q_weight.dtype == torch.float32 and q_weight.numel() == q_size and q_weight.is_contiguous())
        if rot:
            assert rot % 2 == 0 and positions.dtype == torch.int32 and positions.shape[0] == T
            assert inv_freq.dtype == torch.float32 and inv_freq.numel() == rot // 2 and inv_freq.is_contiguous()
        if write:
            assert k_cache.dtype == v_cache.dtype == q.dtype and k_cache.is_contiguous() and v_cache.is_contiguous()
            assert k_cache.numel() == v_cache.numel() == num_pages * page_size * width and slot_map.dtype == torch.int32 and slot_map.shape[0] == T
        self._run("latent_finish", T * (q_size + width) * (4 + q.element_size()) + T * width * q.element_size(), 4 * T * width, None,
                  self.lib.llmrs_latent_finish, self._stream(), _code(q.dtype), _p(sums), sums.stride(0), _p(q), q.stride(0), T, q_size,
                  rank, _p(weight), float(eps), _p(slot_map), _p(k_cache), _p(v_cache), page_size, num_pages, int(write),
                  _p(q_weight), int(rot), _p(positions) if rot else None, _p(inv_freq) if rot else None, float(gain))

    def head_product(self, a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None) -> None:
        """Every head by its own matrix: out[t, h, :] = w[h] @ a[t, h, :] with w [heads, n_out, n_in] (each [out, in]),
        a [T, heads * n_in], out [T, heads * n_out], both in w's type, sums in 32-bit; gate [T, heads] float32: the sums
        of head h are multiplied by sigmoid(gate[t, h]) before the one rounding."""
        H, n_out, n_in = w.shape
        T = a.shape[0]
        assert a.dtype == w.dtype == out.dtype and w.is_contiguous() and a.stride(1) == 1 and out.stride(1) == 1
        assert a.shape[1] == H * n_in and out.shape == (T, H * n_out)
        assert gate is None or (gate.dtype == torch.float32 and gate.shape == (T, H) and gate.stride(1) == 1)
        self._run(f"head_product {T}x{H}x{n_out}x{n_in}", (T * H * (n_in + n_out) + H * n_in * n_out) * a.element_size(),
                  2 * T * H * n_in * n_out, a.dtype, self.lib.llmrs_head_product, self._stream(), _code(a.dtype), _p(a), a.stride(0),
                  _p(w), _p(out), out.stride(0), T, H, n_in, n_out, int(self.allow_mfma), _p(gate), 0 if gate is None else gate.stride(0))

    # out (epilogue) a @ w.T ; a: [M, K] rows may be strided, w: [N, K] dense
    def gemm(self, a, w: torch.Tensor, out: torch.Tensor, epilogue: int = EPI_STORE,
             workspace: Optional[torch.Tensor] = None, leave: Optional[NextNorm] = None, glu=None) -> None:
        """`a` may be `NormedRows`, and `leave` a `NextNorm` (with the += epilogue), where `gemm_defers_norm` holds.
        EPI_GLU_CLAMP (rows of w are gate_0, up_0, gate_1, ...; glu = what `glu_clamp_slot(limit, alpha)` gave): out[m, j] =
        g sigmoid(alpha g) (u + 1) with g = min(gate_j, limit), u = clamp(up_j, -limit, limit), computed on the 32-bit sums,
        in the activation type."""
        assert (glu is not None) == (epilogue == EPI_GLU_CLAMP) and (glu is None or isinstance(glu, int))
        scale = None
        if isinstance(a, NormedRows):
            scale, a = a, a.y
            assert scale.sumsq.dtype == torch.float32 and scale.sumsq.is_contiguous() and scale.sumsq.shape[0] == a.shape[0]
        M, K = a.shape
        N = w.shape[0]
        assert w.shape[1] == K and w.is_contiguous() and a.stride(1) == 1 and out.stride(1) == 1 and a.dtype == w.dtype
        whole = leave is not None and leave.whole
        if leave is not None:
            assert epilogue == EPI_ACCUM_F32 and tuple(leave.y.shape) == (M, N) and leave.y.stride(1) == 1
            assert leave.y.dtype == torch.bfloat16 and leave.weight.dtype == torch.float32 and leave.weight.shape[0] == N
            if not whole:
                assert N < 16384 and leave.sumsq.dtype == torch.float32 and leave.sumsq.is_contiguous()
                assert tuple(leave.sumsq.shape) == (M, self.gemm_next_parts(M, N, K))
        if whole:
            assert a.dtype == torch.bfloat16 and scale is None and self.gemm_norms_whole(M, N, K) and workspace is not None
        elif scale is not None or leave is not None:
            assert a.dtype == torch.bfloat16 and self.gemm_defers_norm(M, N, K)
        want = torch.float32 if epilogue in (EPI_STORE_F32, EPI_ACCUM_F32) else a.dtype
        assert out.dtype == want and out.shape[0] == M and out.shape[1] == (N // 2 if epilogue in _EPI_GATED else N)
        moved = (M * K + N * K) * a.element_size() + out.numel() * out.element_size() * (2 if epilogue == EPI_ACCUM_F32 else 1)
        label = f"gemm {M}x{N}x{K} {'norm+' if scale is not None else ''}{_EPI_NAMES[epilogue]}{('+norm' if whole else '+next') if leave is not None else ''}"
        self._run(label, moved, 2 * M * N * K, a.dtype,
                  self.lib.llmrs_gemm, self._stream(), _code(a.dtype), _p(a), a.stride(0), _p(w), _p(out), out.stride(0),
                  M, N, K, epilogue + (glu or 0), _p(workspace),
                  0 if workspace is None else workspace.numel() * workspace.element_size(), int(self.allow_mfma),
                  None if scale is None else _p(scale.sumsq), 0 if scale is None else scale.sumsq.shape[1],
                  0.0 if scale is None else scale.eps, None if leave is None or whole else _p(leave.sumsq),
                  None if leave is None else _p(leave.y), 0 if leave is None else leave.y.stride(0),
                  None if leave is None else _p(leave.weight), leave.eps if whole else 0.0)

    def glu_clamp_slot(self, limit: float, alpha: float) -> int:
        """Where the kernel library keeps this pair of constants of the clamped gated epilogue on the current device: what
        `gemm(..., EPI_GLU_CLAMP, glu=...)` takes.  Asked for when a feed-forward takes its weights, never inside a
        recording (the first call for a pair writes device memory and waits for the stream)."""
        slot = int(self.lib.llmrs_glu_clamp_slot(self._stream(), float(limit), float(alpha)))
        if slot < 0:
            raise KernelError(self.lib.llmrs_hip_error().decode())
        return slot

    def rope_kv_write(self, qkv, positions, slot_map, inv_freq, rotary_dim, interleaved, k_cache, v_cache,
                      n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv) -> None:
        assert qkv.stride(1) == 1 and positions.dtype == torch.int32
        assert rotary_dim == 0 or (inv_freq.dtype == torch.float32 and inv_freq.shape[0] == rotary_dim // 2)
        if write_kv:
            assert k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype and k_cache.is_contiguous() and v_cache.is_contiguous()
            assert k_cache.numel() == num_pages * n_kv_heads * page_size * head_dim == v_cache.numel()
            assert slot_map.dtype == torch.int32 and slot_map.shape[0] == qkv.shape[0]
        T = qkv.shape[0]
        self._run("rope_kv_write", T * (2 * n_heads + 4 * n_kv_heads) * head_dim * qkv.element_size(),
                  5 * T * (n_heads + n_kv_heads) * rotary_dim, None, self.lib.llmrs_rope_kv_write,
                  self._stream(), _code(qkv.dtype), _p(qkv), qkv.stride(0), _p(positions), _p(slot_map), _p(inv_freq),
                  rotary_dim, int(interleaved), _p(k_cache), _p(v_cache), qkv.shape[0], n_heads, n_kv_heads, head_dim,
                  page_size, num_pages, int(write_kv))

    def qkv_rope_cache(self, x, w, qkv, positions, slot_map, inv_freq, rotary_dim, k_cache, v_cache,
                       n_heads, n_kv_heads, head_dim, page_size, num_pages, write_kv, workspace=None) -> None:
        """qkv = x @ w.T, q and k rotated by adjacent pairs (2i, 2i+1), k and v written to the cache: fused into
        one kernel where the product allows.  Afterwards only the q part of `qkv` is certain to be filled."""
        assert w.shape[0] == (n_heads + 2 * n_kv_heads) * head_dim and w.shape[1] == x.shape[1] and qkv.shape[0] == x.shape[0]
        scale = None
        if isinstance(x, NormedRows):
            scale, x = x, x.y
            assert scale.sumsq.dtype == torch.float32 and scale.sumsq.is_contiguous() and scale.sumsq.shape[0] == x.shape[0]
            assert x.dtype == torch.bfloat16 and self.gemm_defers_norm(x.shape[0], w.shape[0], x.shape[1])
        assert x.stride(1) == 1 and qkv.stride(1) == 1 and w.is_contiguous() and x.dtype == w.dtype == qkv.dtype
        assert rotary_dim == 0 or (inv_freq.dtype == torch.float32 and inv_freq.shape[0] == rotary_dim // 2)
        if write_kv:
            assert k_cache.dtype == x.dtype and k_cache.is_contiguous() and v_cache.is_contiguous()
            assert k_cache.numel() == num_pages * n_kv_heads * page_size * head_dim == v_cache.numel()
        M, K, N = x.shape[0], x.shape[1], w.shape[0]
        self._run(f"gemm {M}x{N}x{K} {'norm+' if scale is not None else ''}qkv+rope+cache", (M * K + N * K + M * N) * x.element_size(), 2 * M * N * K, x.dtype,
                  self.lib.llmrs_qkv_rope_cache,
                  self._stream(), _code(x.dtype), _p(x), x.stride(0), _p(w), _p(qkv), qkv.stride(0), x.shape[0], x.shape[1],
                  _p(positions), _p(slot_map), _p(inv_freq), rotary_dim, _p(k_cache), _p(v_cache), n_heads, n_kv_heads,
                        head_dim, page_size, num_pages, int(write_kv), _p(workspace),
                  0 if workspace is None else workspace.numel() * workspace.element_size(), int(self.allow_mfma),
                  None if scale is None else _p(scale.sumsq), 0 if scale is None else scale.sumsq.shape[1],
                  0.0 if scale is None else scale.eps)

    def attention_split_chunk(self, n_single: int, n_kv_heads: int, head_dim: int, max_seq_len: int, single_keys: int = 0) -> int:
        """Keys per wave that a call with these figures splits its single-token entries by: what a caller that
        records steps into graphs has to key its recordings by, since a recording holds the chunk it was made with
        while the number of keys moves with every step."""
        return int(self.lib.llmrs_attention_split_chunk(int(n_single), int(n_kv_heads), int(head_dim), int(max_seq_len), int(single_keys)))

    def attention(self, q, out, k_cache, v_cache, block_table, token_entry, positions, q_starts, seq_lens,
                  n_heads, n_kv_heads, head_dim, page_size, num_pages, window, scale, scratch=None, max_seq_len=0, n_single=-1,
                  single_keys=0, value_dim=0, distance=None, softcap=0.0, keep_first=0, sink=None, gate=None, gate_per=1) -> None:
        """gate: float32 [T, n_heads * value_dim / gate_per] or None: every gate_per consecutive output features of a token
        are multiplied by the sigmoid of their number (32-bit, before the one rounding).
        sink: float32 [n_heads] or None: the softmax's denominator of head h also holds exp(sink[h]), once for every
        query (a key without a value; not scaled).  single_keys: how many keys the single-token entries see together (windows counted), 0 if unknown.
        value_dim: the width of a value where it is not a key's (0: the same).  distance: (r1, r2), float32 [n_heads]
        each: r1[h] * ln(1 + r2[h] * (i - j)) is taken off the scaled score of query i and key j.  softcap > 0: the
        scaled score s becomes softcap * tanh(s / softcap).  keep_first: with a window, the request's first so many
        keys stay visible to every later query."""
        assert q.stride(1) == 1 and out.stride(1) == 1 and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype
        assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
        v_dim = int(value_dim) or head_dim
        assert k_cache.numel() == num_pages * n_kv_heads * page_size * head_dim and v_cache.numel() == num_pages * n_kv_heads * page_size * v_dim
        if v_dim != head_dim or distance is not None or softcap > 0 or (keep_first > 0 and window > 0) or sink is not None or gate is not None:
            return self._attention_ext(q, out, k_cache, v_cache, block_table, token_entry, positions, q_starts, seq_lens, n_heads,
                                       n_kv_heads, head_dim, page_size, num_pages, window, scale, scratch, max_seq_len, n_single,
                                       single_keys, v_dim, distance, softcap, keep_first, sink, gate, gate_per)
        T = q.shape[0]
        assert token_entry.shape[0] == T and positions.shape[0] == T and out.shape[0] == T
        moved = flops = 0
        if self.times is not None:      # what the call has to read depends on the step: ask the device (timing mode only)
            keys = int(seq_lens.sum().item())
            seen = int((positions + 1).sum().item()) if window <= 0 else int((positions + 1).clamp(max=window).sum().item())
            moved = (2 * keys * n_kv_heads + 2 * T * n_heads) * head_dim * q.element_size()
            flops = 4 * seen * n_heads * head_dim
        self._run(f"attention {T} tokens" + (" (decode)" if n_single == block_table.shape[0] else ""), moved, flops, q.dtype,
                  self.lib.llmrs_attention,
                  self._stream(), _code(q.dtype), _p(q), q.stride(0), _p(out), out.stride(0), _p(k_cache), _p(v_cache),
                  _p(block_table), block_table.shape[1], _p(token_entry), _p(positions), _p(q_starts), _p(seq_lens),
                  block_table.shape[0], T, n_heads, n_kv_heads, head_dim, page_size, num_pages, window, scale,
                  _p(scratch), 0 if scratch is None else scratch.numel() * scratch.element_size(), int(max_seq_len),
                  int(n_single), int(single_keys), int(self.allow_mfma))

    def _attention_ext(self, q, out, k_cache, v_cache, block_table, token_entry, positions, q_starts, seq_lens, n_heads,
                       n_kv_heads, head_dim, page_size, num_pages, window, scale, scratch, max_seq_len, n_single, single_keys,
                       v_dim, distance, softcap=0.0, keep_first=0, sink=None, gate=None, gate_per=1) -> None:
        T = q.shape[0]
        assert gate is None or (gate.dtype == torch.float32 and gate.stride(1) == 1 and gate.shape[0] == T and gate_per >= 1
                                and (n_heads * v_dim) % gate_per == 0 and gate.shape[1] == n_heads * v_dim // gate_per)
        assert sink is None or (sink.dtype == torch.float32 and sink.numel() == n_heads and sink.is_contiguous())
        assert token_entry.shape[0] == T and positions.shape[0] == T and out.shape[0] == T
        r1 = r2 = None
        if distance is not None:
            r1, r2 = distance
            assert r1.dtype == r2.dtype == torch.float32 and r1.numel() == r2.numel() == n_heads and r1.is_contiguous() and r2.is_contiguous()
        moved = flops = 0
        if self.times is not None:
            keys = int(seq_lens.sum().item())
            seen = int((positions + 1).sum().item()) if window <= 0 else int((positions + 1).clamp(max=window + keep_first).sum().item())
            moved = (keys * n_kv_heads * (head_dim + v_dim) + T * n_heads * (head_dim + v_dim)) * q.element_size()
            flops = 2 * seen * n_heads * (head_dim + v_dim)
        self._run(f"attention {T} tokens" + (" (decode)" if n_single == block_table.shape[0] else ""), moved, flops, q.dtype,
                  self.lib.llmrs_attention_ext,
                  self._stream(), _code(q.dtype), _p(q), q.stride(0), _p(out), out.stride(0), _p(k_cache), _p(v_cache),
                  _p(block_table), block_table.shape[1], _p(token_entry), _p(positions), _p(q_starts), _p(seq_lens),
                  block_table.shape[0], T, n_heads, n_kv_heads, head_dim, page_size, num_pages, window, scale,
                  _p(scratch), 0 if scratch is None else scratch.numel() * scratch.element_size(), int(max_seq_len),
                  int(n_single), int(single_keys), int(self.allow_mfma), v_dim, _p(r1), _p(r2), float(softcap), int(keep_first), _p(sink),
                  _p(gate), 0 if gate is None else gate.stride(0), int(gate_per))

    # out[i, :] = weight * groupnorm(sum_s w_in[s] * x[s][rows[i] or i, :]); x: [T, D] or [S, T, D] float32
    def group_rmsnorm(self, out: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float, groups: int,
                      rows: Optional[torch.Tensor] = None, w_in: Optional[torch.Tensor] = None,
                      zero: Optional[torch.Tensor] = None, combined: Optional[torch.Tensor] = None, mix=None) -> None:
        """The RMS norm in `groups` equal consecutive parts of the row.  `x` with three dimensions is several streams,
        combined with the weights `w_in` (None: summed) before the norm.  `zero` [n, D] float32 is cleared on the way,
        `combined` [n, D] float32 gets the combined rows.  `mix` = (mix [S, S], w_out [S], y [n, D]): `streams_mix`
        of these runs on x first, in the same launch (every row, no `rows`); y may be `zero`."""
        assert x.dtype == torch.float32 and weight.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous()
        S = x.shape[0] if x.dim() == 3 else 1
        D, n = x.shape[-1], out.shape[0]
        assert out.shape[1] == D == weight.shape[0]
        assert (rows is None and n == x.shape[-2]) or (rows is not None and rows.dtype == torch.int32 and rows.shape[0] == n)
        assert w_in is None or (w_in.dtype == torch.float32 and w_in.numel() == S)
        for extra in (zero, combined):
            assert extra is None or (extra.dtype == torch.float32 and extra.is_contiguous() and tuple(extra.shape) == (n, D))
        m = w_out = y = None
        if mix is not None:
            m, w_out, y = mix
            assert rows is None and x.dim() == 3 and m.dtype == w_out.dtype == y.dtype == torch.float32
            assert tuple(m.shape) == (S, S) and m.is_contiguous() and w_out.numel() == S and y.is_contiguous() and tuple(y.shape) == (n, D)
        traffic = n * D * (4 * S + out.element_size()) + D * 4 + (n * D * 4 * (S + 1) if mix is not None else 0)
        self._run(f"group_rmsnorm {n}x{D}" + (f" of {S} streams" if S > 1 else "") + (" after their mix" if mix is not None else ""),
                  traffic, (2 * S + 5 + (2 * S * S if mix is not None else 0)) * n * D, None, self.lib.llmrs_group_rmsnorm,
                  self._stream(), _code(out.dtype), _p(out), _p(x),
                  x.stride(0) if x.dim() == 3 else 0, S, _p(w_in), _p(weight), _p(rows), n, D, int(groups), float(eps),
                  _p(zero), _p(combined), _p(m), _p(w_out), _p(y))

    # x[r] = sum_s mix[s, r] * x[s] + w_out[r] * y, all streams at once from the old ones; x: [S, T, D] float32
    def streams_mix(self, x: torch.Tensor, mix: torch.Tensor, w_out: torch.Tensor, y: torch.Tensor) -> None:
        assert x.dim() == 3 and x.dtype == y.dtype == mix.dtype == w_out.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous()
        S = x.shape[0]
        assert tuple(mix.shape) == (S, S) and mix.is_contiguous() and w_out.numel() == S and y.numel() == x[0].numel()
        self._run(f"streams_mix {S}x{y.shape[0]}x{y.shape[1]}", (2 * S + 1) * y.numel() * 4, 2 * S * S * y.numel(), None,
                  self.lib.llmrs_streams_mix, self._stream(), _p(x), x.stride(0), S, _p(mix), _p(w_out), _p(y), y.numel())

    # x[s] = x[0] for every s
    def streams_copy_first(self, x: torch.Tensor) -> None:
        assert x.dim() == 3 and x.dtype == torch.float32 and x.is_contiguous()
        self._run("streams_copy_first", (x.shape[0] + 1) * x[0].numel() * 4, 0, None,
                  self.lib.llmrs_streams_copy_first, self._stream(), _p(x), x.stride(0), x.shape[0], x[0].numel())

    def qkv_finish(self, sums: torch.Tensor, bias: Optional[torch.Tensor], q: torch.Tensor, slot_map, k_cache, v_cache,
                   n_heads: int, n_kv_heads: int, head_dim: int, v_dim: int, page_size: int, num_pages: int, write_kv: bool,
                   eps: float, positions: Optional[torch.Tensor] = None, inv_freq: Optional[torch.Tensor] = None, rotary_dim: int = 0,
                   q_weight: Optional[torch.Tensor] = None, k_weight: Optional[torch.Tensor] = None, gain: float = 1.0, conv=None) -> None:
        """sums [T, q | k | v] float32 -> q [T, heads * head_dim] (activation type) and the cache's pages: biases
        added, q and k divided by their root mean square over the head (eps > 0) and multiplied by q_weight / k_weight
        [head_dim] (if given), then (rotary_dim > 0) their features (2i, 2i + 1) turned by positions[t] * inv_freq[i],
        cosine and sine times `gain`; one rounding on the way out.
        conv = (taps [columns, K] float32, state [slots, >= (K - 1) * columns] float32 or None when K == 1, q_starts, slots,
        token_entry): every column first passes a causal convolution over its K taps, the last tap the token's own; rows
        before an entry's first token come from the request's state (which `conv_state_update` brings up to date afterwards)."""
        taps = state = q_starts = slots = token_entry = None
        n_taps = n_entries = 0
        if conv is not None:
            taps, state, q_starts, slots, token_entry = conv
            n_taps, n_entries = taps.shape[1], slots.numel()
            assert taps.dtype == torch.float32 and taps.is_contiguous() and taps.shape[0] == sums.shape[1]
            assert q_starts.dtype == slots.dtype == token_entry.dtype == torch.int32 and token_entry.numel() == sums.shape[0]
            assert n_taps == 1 or (state is not None and state.dtype == torch.float32 and state.stride(-1) == 1
                                   and state.shape[1] >= (n_taps - 1) * sums.shape[1])
        for w in (q_weight, k_weight):
            assert w is None or (w.dtype == torch.float32 and w.numel() == head_dim and w.is_contiguous() and eps > 0)
        if rotary_dim:
            assert positions.dtype == torch.int32 and positions.shape[0] == sums.shape[0] and inv_freq.dtype == torch.float32
            assert inv_freq.shape[0] == rotary_dim // 2 and inv_freq.is_contiguous() and rotary_dim % 2 == 0 and rotary_dim <= head_dim
        assert sums.dtype == torch.float32 and sums.stride(1) == 1 and q.stride(1) == 1 and q.shape[0] == sums.shape[0]
        width = (n_heads + n_kv_heads) * head_dim + n_kv_heads * v_dim
        assert sums.shape[1] == width and (bias is None or (bias.dtype == torch.float32 and bias.numel() == width and bias.is_contiguous()))
        if write_kv:
            assert k_cache.dtype == v_cache.dtype == q.dtype and k_cache.is_contiguous() and v_cache.is_contiguous()
            assert k_cache.numel() == num_pages * n_kv_heads * page_size * head_dim and v_cache.numel() == num_pages * n_kv_heads * page_size * v_dim
            assert slot_map.dtype == torch.int32 and slot_map.shape[0] == sums.shape[0]
        T = sums.shape[0]
        self._run("qkv_finish", T * width * (4 + q.element_size()), 4 * T * width, None, self.lib.llmrs_qkv_finish,
                  self._stream(), _code(q.dtype), _p(sums), sums.stride(0), _p(bias), _p(q), q.stride(0), _p(slot_map),
                  _p(k_cache), _p(v_cache), T, n_heads, n_kv_heads, head_dim, v_dim, page_size, num_pages, int(write_kv), float(eps),
                  _p(positions) if rotary_dim else None, _p(inv_freq) if rotary_dim else None, int(rotary_dim),
                  _p(q_weight), _p(k_weight), float(gain), _p(taps), int(n_taps), _p(state) if n_taps > 1 else None,
                  state.stride(0) if n_taps > 1 else 0, _p(q_starts), _p(slots), _p(token_entry), int(n_entries))

    def add_bias_rows(self, rows: torch.Tensor, bias: torch.Tensor) -> None:
        """rows[t, :] += bias; both float32."""
        assert rows.dtype == bias.dtype == torch.float32 and rows.stride(1) == 1 and bias.numel() == rows.shape[1] and bias.is_contiguous()
        self._run(f"add_bias {rows.shape[0]}x{rows.shape[1]}", rows.numel() * 8, rows.numel(), None,
                  self.lib.llmrs_add_bias_rows, self._stream(), _p(rows), rows.stride(0), _p(bias), rows.shape[0], rows.shape[1])

    def linear_scan(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, q_starts, slots, heads: int,
                    qk_heads: int, dk: int, dv: int, out: torch.Tensor, decay: Optional[torch.Tensor] = None,
                    g: Optional[torch.Tensor] = None, beta: Optional[torch.Tensor] = None, gates=None, v_cols: int = 0) -> None:
        """Per head a matrix S [dk, dv] carried from token to token: S <- decay S (decay [heads], or g [T, heads * dk] a
        key channel); u = beta (v - S^T k) (beta [T, heads]; None: u = v); S <- S + k u^T; out = S^T q.  q, k
        [T, qk_heads * dk], v and out [T, heads * dv], all float32 with unit column stride; state [slots, >= heads * dk * dv]
        float32, laid out [heads][dv][dk] (a value channel's key channels side by side), read at an entry's first token
        and left at its last.  gates = (decay, take), [T, heads] each: S <- decay S + take k v^T, gates that move with the
        token.  v_cols (< dv): v holds only so many columns a head, [T, heads * v_cols]; the others are written with 1 in
        v's place, so that a column of S past v_cols is the gated sum of the keys themselves."""
        T = q.shape[0]
        tdecay, ttake = gates if gates is not None else (None, None)
        v_cols = int(v_cols) or dv
        for t in (q, k, v, out, g, beta, tdecay, ttake):
            assert t is None or (t.dtype == torch.float32 and t.stride(1) == 1 and t.shape[0] == T)
        assert q.shape[1] == k.shape[1] == qk_heads * dk and v.shape[1] == heads * v_cols and out.shape[1] == heads * dv and 0 < v_cols <= dv
        assert gates is None or (tdecay.shape[1] == ttake.shape[1] == heads and tdecay.stride(0) == ttake.stride(0)
                                 and decay is None and g is None and beta is None)
        assert state.dtype == torch.float32 and state.stride(-1) == 1 and state.shape[1] >= heads * dk * dv
        assert q_starts.dtype == slots.dtype == torch.int32 and q_starts.numel() == slots.numel() + 1
        assert decay is None or (decay.dtype == torch.float32 and decay.numel() == heads and decay.is_contiguous())
        assert g is None or g.shape[1] == heads * dk
        assert beta is None or beta.shape[1] == heads
        kind = ("delta" if beta is not None else "decay") + (" by channel" if g is not None else " by token" if gates is not None else "")
        self._run(f"linear_scan {T}x{heads}x{dk}x{dv} {kind}", T * (2 * qk_heads * dk + (heads * dk if g is not None else 0) + 2 * heads * dv) * 4
                  + slots.numel() * heads * dk * dv * 8, (7 if beta is not None else 5) * T * heads * dk * dv, None,
                  self.lib.llmrs_linear_scan, self._stream(), _p(q), q.stride(0), _p(k), k.stride(0), _p(v), v.stride(0),
                  _p(g), 0 if g is None else g.stride(0), _p(decay), _p(beta), 0 if beta is None else beta.stride(0),
                  _p(state), state.stride(0), _p(q_starts), _p(slots), slots.numel(), T, heads, qk_heads, dk, dv, _p(out), out.stride(0),
                  _p(tdecay), _p(ttake), 0 if gates is None else tdecay.stride(0), v_cols)

    def exp_gates(self, gi: torch.Tensor, gf: torch.Tensor, bias_i, bias_f, cap: float, m_state: torch.Tensor, q_starts, slots,
                  decay: torch.Tensor, take: torch.Tensor, floor: torch.Tensor) -> None:
        """The gates of a matrix memory with exponential gates, per (token, head), float32: with i = cap tanh((gi + bias_i)
        / cap), f = log sigmoid(cap tanh((gf + bias_f) / cap)) and the running maximum m_t = max(f + m_(t-1), i) carried in
        m_state [slots, heads] (read at an entry's first token, left at its last): decay = exp(f + m_(t-1) - m_t),
        take = exp(i - m_t), floor = exp(-m_t).  gi, gf [T, heads] (columns of a product's sums, equal row strides)."""
        T, H = gi.shape
        for t in (gi, gf, decay, take, floor):
            assert t.dtype == torch.float32 and t.stride(1) == 1 and tuple(t.shape) == (T, H)
        assert gi.stride(0) == gf.stride(0) and decay.stride(0) == take.stride(0) == floor.stride(0)
        for b in (bias_i, bias_f):
            assert b is None or (b.dtype == torch.float32 and b.numel() == H and b.is_contiguous())
        assert m_state.dtype == torch.float32 and m_state.stride(-1) == 1 and m_state.shape[1] >= H
        assert q_starts.dtype == slots.dtype == torch.int32 and q_starts.numel() == slots.numel() + 1
        self._run(f"exp_gates {T}x{H}", T * H * 20, 40 * T * H, None, self.lib.llmrs_exp_gates, self._stream(), _p(gi), _p(gf), gi.stride(0),
                  _p(bias_i), _p(bias_f), float(cap), _p(m_state), m_state.stride(0), _p(q_starts), _p(slots), slots.numel(), T, H,
                  _p(decay), _p(take), _p(floor), decay.stride(0))

    def qkv_whole(self, sums: torch.Tensor, q_cols: int, k_cols: int, v_cols: int, q_weight, k_weight, eps: float,
                  first: Optional[torch.Tensor] = None, lam: Optional[torch.Tensor] = None, keep: Optional[torch.Tensor] = None) -> None:
        """In place on sums [T, q | k | v] float32: q (k) RMS-normed over the whole projection and multiplied by q_weight
        [q_cols] (k_weight [k_cols]; None: left as it is); v <- (1 - lam) v + lam first with first [T, v_cols] float32 and
        lam one number on the device, or (keep [T, v_cols] given instead) v copied out for a later layer to mix with."""
        T = sums.shape[0]
        assert sums.dtype == torch.float32 and sums.stride(1) == 1 and sums.shape[1] >= q_cols + k_cols + v_cols
        for w, n in ((q_weight, q_cols), (k_weight, k_cols)):
            assert w is None or (w.dtype == torch.float32 and w.numel() == n and w.is_contiguous())
        for t in (first, keep):
            assert t is None or (t.dtype == torch.float32 and t.stride(1) == 1 and tuple(t.shape) == (T, v_cols))
        assert first is None or (lam is not None and lam.dtype == torch.float32 and lam.numel() == 1 and keep is None)
        self._run("qkv_whole", T * (q_cols + k_cols + v_cols) * 8, 4 * T * (q_cols + k_cols + v_cols), None, self.lib.llmrs_qkv_whole,
                  self._stream(), _p(sums), sums.stride(0), T, q_cols, k_cols, v_cols, _p(q_weight), _p(k_weight), float(eps),
                  _p(first), 0 if first is None else first.stride(0), _p(lam), _p(keep), 0 if keep is None else keep.stride(0))

    def silu_columns(self, x: torch.Tensor, col0: int, n: int) -> None:
        """x[:, col0:col0 + n] <- silu of itself; x float32 with unit column stride."""
        assert x.dtype == torch.float32 and x.stride(1) == 1 and 0 <= col0 and col0 + n <= x.shape[1]
        self._run(f"silu {x.shape[0]}x{n}", x.shape[0] * n * 8, 4 * x.shape[0] * n, None,
                  self.lib.llmrs_silu_columns, self._stream(), _p(x), x.stride(0), x.shape[0], int(col0), int(n))

    def delta_prepare(self, q: torch.Tensor, k: torch.Tensor, a: torch.Tensor, b: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor,
                      heads: int, qk_heads: int, dk: int, unit_eps: float) -> None:
        """In place, float32: q, k [T, qk_heads * dk] made unit vectors per head (x / sqrt(sum x^2 + unit_eps)), q also
        times dk^(-1/2); a [T, heads * dk] <- exp(-exp(A_log[h]) softplus(a + dt_bias)); b [T, heads] <- sigmoid(b)."""
        T = q.shape[0]
        for t in (q, k, a, b):
            assert t.dtype == torch.float32 and t.stride(1) == 1 and t.shape[0] == T
        assert q.shape[1] == k.shape[1] == qk_heads * dk and a.shape[1] == heads * dk and b.shape[1] == heads
        assert A_log.dtype == dt_bias.dtype == torch.float32 and A_log.numel() == heads and dt_bias.numel() == heads * dk
        assert A_log.is_contiguous() and dt_bias.is_contiguous()
        self._run(f"delta_prepare {T}x{heads}x{dk}", T * (2 * qk_heads + heads) * dk * 8, 8 * T * (2 * qk_heads + heads) * dk, None,
                  self.lib.llmrs_delta_prepare, self._stream(), _p(q), q.stride(0), _p(k), k.stride(0), _p(a), a.stride(0),
                  _p(b), b.stride(0), _p(A_log), _p(dt_bias), T, heads, qk_heads, dk, float(unit_eps))

    def gated_rmsnorm(self, out: torch.Tensor, x: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, group: int, eps: float,
                      floor: Optional[torch.Tensor] = None, x_scale: float = 1.0, den_add: float = 0.0) -> None:
        """out[t, c] = y[t, c] / sqrt(mean of y^2 over c's group of `group` columns + eps) * weight[c % len(weight)] *
        sigmoid(gate[t, c]); x, gate float32, weight float32 of a group's or a row's length.  y = x; or, with floor
        [T, groups] float32, x has one more column n behind each group (x [T, groups * (group + 1)]) and
        y = x_scale x / (max(x_scale |n|, floor) + den_add)."""
        T, W = gate.shape
        stride = group + (1 if floor is not None else 0)
        assert x.dtype == gate.dtype == weight.dtype == torch.float32 and x.stride(1) == gate.stride(1) == out.stride(1) == 1
        assert out.shape == gate.shape and W % group == 0 and x.shape == (T, W // group * stride) and weight.numel() in (group, W) and weight.is_contiguous()
        assert floor is None or (floor.dtype == torch.float32 and floor.stride(1) == 1 and tuple(floor.shape) == (T, W // group))
        self._run(f"gated_rmsnorm {T}x{W}", T * W * (8 + out.element_size()), 8 * T * W, None,
                  self.lib.llmrs_gated_rmsnorm, self._stream(), _code(out.dtype), _p(x), x.stride(0), _p(gate), gate.stride(0),
                  _p(weight), weight.numel(), T, W // group, int(group), float(eps), _p(out), out.stride(0), stride, _p(floor),
                  0 if floor is None else floor.stride(0), float(x_scale), float(den_add))

    def rmsnorm_sum(self, out: torch.Tensor, inputs, coef: float, eps: float) -> None:
        """out += coef * sum of rmsnorm(x + bias) * weight over `inputs`, one or two (x [T, D], bias [D] or None,
        weight [D]); everything float32 and contiguous."""
        assert 1 <= len(inputs) <= 2 and out.dtype == torch.float32 and out.is_contiguous()
        T, D = out.shape
        flat = []
        for x, bias, weight in inputs:
            assert x.dtype == weight.dtype == torch.float32 and x.is_contiguous() and tuple(x.shape) == (T, D) and weight.numel() == D
            assert bias is None or (bias.dtype == torch.float32 and bias.numel() == D)
            flat += [_p(x), _p(bias), _p(weight)]
        flat += [None] * (6 - len(flat))
        self._run(f"rmsnorm_sum {T}x{D} of {len(inputs)}", T * D * 4 * (2 + len(inputs)), 6 * len(inputs) * T * D, None,
                  self.lib.llmrs_rmsnorm_sum, self._stream(), _p(out), *flat, T, D, float(coef), float(eps))

    def route_topk(self, logits: torch.Tensor, weights: torch.Tensor, top: int, renormalize: bool = False, score: str = "softmax",
                   correction: Optional[torch.Tensor] = None, scale: float = 1.0) -> None:
        """weights[t, e] = softmax(logits[t])[e] for the `top` experts with the largest scores (of equal ones the lower
        index), 0 for the others; with `renormalize` divided by the chosen scores' sum.  Both float32 [T, experts].
        score = "sigmoid": an expert's score is sigmoid(logit); the choice goes by score + correction [experts] (None:
        by the score), the weight is the score without it (with `renormalize` divided by the chosen scores' sum + 1e-20),
        times scale."""
        assert logits.dtype == weights.dtype == torch.float32 and logits.stride(1) == weights.stride(1) == 1 and logits.shape == weights.shape
        T, E = logits.shape
        kind = {"softmax": 0, "sigmoid": 1}[score]
        assert correction is None or (kind == 1 and correction.dtype == torch.float32 and correction.numel() == E and correction.is_contiguous())
        assert kind == 1 or scale == 1.0
        self._run(f"route_topk {T}x{E}", T * E * 8, 8 * T * E, None, self.lib.llmrs_route_topk, self._stream(), _p(logits),
                  logits.stride(0), _p(weights), weights.stride(0), T, E, int(top), int(bool(renormalize)), kind, _p(correction), float(scale))

    def route_counts(self, weights: torch.Tensor, counts: torch.Tensor) -> None:
        """counts[e] = how many tokens chose expert e (weights[t, e] > 0); weights float32 [T, E], counts int32 [E]."""
        assert weights.dtype == torch.float32 and weights.stride(1) == 1 and counts.dtype == torch.int32 and counts.numel() == weights.shape[1]
        self._run("route_counts", weights.numel() * 4, 0, None, self.lib.llmrs_route_counts, self._stream(), _p(weights), weights.stride(0),
                  weights.shape[0], weights.shape[1], _p(counts))

    def route_rows(self, weights: torch.Tensor, counts: torch.Tensor, row_token: torch.Tensor, row_weight: torch.Tensor, row_of: torch.Tensor) -> None:
        """The chosen (token, expert) pairs expert by expert, each expert's in the order of their tokens: row_token and
        row_weight [rows], row_of [T, E] (the pair's row, or -1)."""
        T, E = weights.shape
        assert row_token.dtype == row_of.dtype == torch.int32 and row_weight.dtype == torch.float32 and row_of.is_contiguous() and tuple(row_of.shape) == (T, E)
        self._run("route_rows", weights.numel() * 8, 0, None, self.lib.llmrs_route_rows, self._stream(), _p(weights), weights.stride(0), T, E,
                  _p(counts), _p(row_token), _p(row_weight), _p(row_of))

    def gather_rows(self, out: torch.Tensor, x: torch.Tensor, rows: torch.Tensor) -> None:
        """out[r] = x[rows[r]]; rows int32."""
        assert out.dtype == x.dtype and out.stride(1) == x.stride(1) == 1 and out.shape[1] == x.shape[1] and rows.dtype == torch.int32 and rows.numel() == out.shape[0]
        self._run(f"gather_rows {out.shape[0]}x{out.shape[1]}", 2 * out.numel() * out.element_size(), 0, None, self.lib.llmrs_gather_rows,
                  self._stream(), _code(out.dtype), _p(out), out.stride(0), _p(x), x.stride(0), _p(rows), out.shape[0], out.shape[1])

    def combine_rows(self, h: torch.Tensor, y: torch.Tensor, row_of: torch.Tensor) -> None:
        """h[t] += the sum of y[row_of[t, e]] over the experts e with row_of[t, e] >= 0, in ascending e; float32."""
        assert h.dtype == y.dtype == torch.float32 and h.stride(1) == y.stride(1) == 1 and h.shape[1] == y.shape[1]
        assert row_of.dtype == torch.int32 and row_of.is_contiguous() and row_of.shape[0] == h.shape[0]
        self._run(f"combine_rows {h.shape[0]}x{h.shape[1]}", (y.numel() + 2 * h.numel()) * 4, y.numel(), None, self.lib.llmrs_combine_rows,
                  self._stream(), _p(h), h.stride(0), _p(y), y.stride(0), _p(row_of), h.shape[0], row_of.shape[1], h.shape[1])

    def act_weight(self, out: torch.Tensor, up: torch.Tensor, weights: Optional[torch.Tensor], ff: int, activation: str = "relu2",
                   limit: float = 0.0, alpha: float = 1.0) -> None:
        """out[t, c] = act * (weights[t, c // ff] if weights is given); up, weights float32.  "relu2": act =
        relu(up[t, c])^2.  "clamped_glu": up holds (gate, up) side by side, [T, 2 N]; with g = min(up[t, 2c], limit) and
        u = clamp(up[t, 2c + 1], -limit, limit), act = g sigmoid(alpha g) (u + 1)."""
        T, N = out.shape
        kind = {"relu2": 0, "clamped_glu": 1}[activation]
        assert up.dtype == torch.float32 and up.stride(1) == 1 and up.shape == (T, N * (2 if kind == 1 else 1)) and out.stride(1) == 1 and N % ff == 0
        assert weights is None or (weights.dtype == torch.float32 and weights.stride(1) == 1 and tuple(weights.shape) == (T, N // ff))
        self._run(f"act_weight {T}x{N}", T * N * (4 * (kind + 1) + out.element_size()), (3 + 8 * kind) * T * N, None,
                  self.lib.llmrs_act_weight, self._stream(), _code(out.dtype), _p(up), up.stride(0), _p(weights),
                  0 if weights is None else weights.stride(0), int(ff), T, N, kind, _p(out), out.stride(0), float(limit), float(alpha))

    def scan_carry_floats(self, n_tokens: int, n_entries: int, longest: int, per_place: int) -> int:
        """Room (in floats) for what the chunks of a recurrence hand on, `per_place` floats for each chunk's place;
        0 when no entry of the step is long enough to be cut."""
        return int(self.lib.llmrs_scan_places(n_tokens, n_entries)) * per_place if longest > self.scan_chunk else 0

    def scan_set_chunk(self, tokens: int) -> None:
        """The chunk length of the recurrences: 32 or 64 tokens, or 0 for the launcher's own choice."""
        if self.lib.llmrs_scan_set_chunk(int(tokens)):
            raise KernelError(self.lib.llmrs_hip_error().decode())

    def mingru_scan(self, sums: torch.Tensor, bias_z, bias_c, state: torch.Tensor, q_starts, slots, width: int, out: torch.Tensor,
                    longest: int = 0, carry: Optional[torch.Tensor] = None) -> None:
        """sums [T, gate | candidate | output gate] float32; state [slots, width] float32, read and left; out [T, width].
        longest: the most tokens an entry brings; with `carry` (scan_carry_floats(T, entries, longest, 2 * width)
        floats) entries longer than a chunk run in chunks side by side."""
        assert sums.dtype == torch.float32 and sums.stride(1) == 1 and sums.shape[1] == 3 * width and out.stride(1) == 1
        assert state.dtype == torch.float32 and state.stride(-1) == 1 and state.shape[1] >= width and out.shape == (sums.shape[0], width)
        assert q_starts.dtype == slots.dtype == torch.int32 and q_starts.numel() == slots.numel() + 1
        for b in (bias_z, bias_c):
            assert b is None or (b.dtype == torch.float32 and b.numel() == width)
        T = sums.shape[0]
        assert carry is None or (carry.dtype == torch.float32 and carry.is_contiguous()
                                 and carry.numel() >= self.scan_carry_floats(T, slots.numel(), longest, 2 * width))
        self._run(f"mingru_scan {T}x{width}", T * width * (12 + out.element_size()), 12 * T * width, None, self.lib.llmrs_mingru_scan,
                  self._stream(), _code(out.dtype), _p(sums), sums.stride(0), _p(bias_z), _p(bias_c), _p(state), state.stride(0),
                  _p(q_starts), _p(slots), slots.numel(), width, _p(out), out.stride(0), int(longest), _p(carry))

    def causal_conv_silu(self, sums: torch.Tensor, taps: torch.Tensor, bias, state: torch.Tensor, q_starts, slots, token_entry,
                         channels: int, out: torch.Tensor) -> None:
        """out[t, c] = silu(bias[c] + sum_j taps[c, j] * x[t - (K - 1 - j), c]) over the first `channels` columns x of
        sums (float32); state [slots, >= (K - 1) * channels] float32 holds each request's last K - 1 inputs and is brought up to date."""
        K = taps.shape[1]
        assert sums.dtype == taps.dtype == state.dtype == torch.float32 and sums.stride(1) == 1 and taps.is_contiguous() and taps.shape[0] == channels
        assert state.stride(-1) == 1 and state.shape[1] >= (K - 1) * channels and out.shape == (sums.shape[0], channels) and out.stride(1) == 1
        assert q_starts.dtype == slots.dtype == token_entry.dtype == torch.int32 and token_entry.numel() == sums.shape[0]
        T = sums.shape[0]
        self._run(f"causal_conv {T}x{channels}", T * channels * (4 + out.element_size()), 2 * K * T * channels, None,
                  self.lib.llmrs_causal_conv_silu, self._stream(), _code(out.dtype), _p(sums), sums.stride(0), _p(taps), _p(bias),
                  _p(state), state.stride(0), _p(q_starts), _p(slots), _p(token_entry), slots.numel(), T, channels, K, _p(out), out.stride(0))

    def selective_scan(self, x: torch.Tensor, bc: torch.Tensor, off_b: int, off_c: int, dt: torch.Tensor, dt_bias, A: torch.Tensor,
                       D: torch.Tensor, gate: torch.Tensor, state: torch.Tensor, q_starts, slots, out: torch.Tensor,
                       ypart: Optional[torch.Tensor] = None, longest: int = 0, carry: Optional[torch.Tensor] = None) -> None:
        """S[c, n] <- exp(step_c A[c, n]) S[c, n] + step_c x_c B_n, y_c = sum_n S[c, n] C_n + D_c x_c, out = y * silu(gate),
        step = softplus(dt + dt_bias); x, bc (B at column off_b, C at off_c) and out in the activation type, dt and gate
        float32 [T, channels], A [states, channels] (transposed), state [slots, >= states * channels] float32 (state by
        channel), read and left.  longest: the most tokens an
        entry brings; with `carry` (scan_carry_floats(T, entries, longest, (states + 1) * channels) floats) entries
        longer than a chunk run in chunks side by side."""
        N, C = A.shape
        T = x.shape[0]
        assert x.dtype == bc.dtype == out.dtype and x.stride(1) == bc.stride(1) == out.stride(1) == 1 and x.shape[1] == C
        assert dt.dtype == gate.dtype == A.dtype == D.dtype == state.dtype == torch.float32 and A.is_contiguous() and D.numel() == C
        assert dt.stride(1) == gate.stride(1) == 1 and dt.shape == (T, C) and gate.shape == (T, C) and out.shape == (T, C)
        assert state.stride(-1) == 1 and state.shape[1] >= C * N and (dt_bias is None or (dt_bias.dtype == torch.float32 and dt_bias.numel() == C))
        assert ypart is None or (ypart.dtype == torch.float32 and ypart.is_contiguous() and ypart.numel() >= T * C)
        assert bc.shape[0] == T and q_starts.dtype == slots.dtype == torch.int32 and q_starts.numel() == slots.numel() + 1
        assert carry is None or (carry.dtype == torch.float32 and carry.is_contiguous()
                                 and carry.numel() >= self.scan_carry_floats(T, slots.numel(), longest, (N + 1) * C))
        self._run(f"selective_scan {T}x{C}x{N}", T * (C * (8 + 2 * x.element_size()) + 2 * N * x.element_size()) + slots.numel() * C * N * 8,
                  7 * T * C * N, None,
                  self.lib.llmrs_selective_scan, self._stream(), _code(x.dtype), _p(x), x.stride(0), _p(bc), bc.stride(0), int(off_b),
                  int(off_c), _p(dt), dt.stride(0), _p(dt_bias), _p(A), _p(D), _p(gate), gate.stride(0), _p(state), state.stride(0),
                  _p(ypart), _p(q_starts), _p(slots), slots.numel(), T, C, N, _p(out), out.stride(0), int(longest), _p(carry))

    def argmax_rows(self, logits: torch.Tensor, out: torch.Tensor, scratch: Optional[torch.Tensor] = None) -> None:
        """`scratch`: 256 bytes per row let several blocks share a long row."""
        assert logits.dtype == torch.float32 and logits.stride(1) == 1 and out.dtype == torch.int32
        self._run("argmax", logits.numel() * 4, 0, None,
                  self.lib.llmrs_argmax_rows, self._stream(), _p(logits), logits.stride(0), logits.shape[0],
                  logits.shape[1], _p(out), _p(scratch), 0 if scratch is None else scratch.numel() * scratch.element_size())

    def place_ids(self, tokens: torch.Tensor, rows: torch.Tensor, sources: torch.Tensor, ids: torch.Tensor, vocab: int) -> None:
        """tokens[rows[i]] = ids[sources[i]]: what a step sampled goes into the next step's tokens on the device."""
        assert all(t.dtype == torch.int32 and t.is_contiguous() for t in (tokens, rows, sources, ids)) and rows.numel() == sources.numel()
        self._run("place_ids", rows.numel() * 12, 0, None,
                  self.lib.llmrs_place_ids, self._stream(), _p(tokens), tokens.numel(), _p(rows), _p(sources), _p(ids),
                  ids.numel(), rows.numel(), int(vocab))

    # words[i] = uniform (float bits), temperature (float bits), top_k, top_p (float bits) of row i
    def sample_rows(self, logits: torch.Tensor, words: torch.Tensor, out: torch.Tensor) -> None:
        assert logits.dtype == torch.float32 and logits.stride(1) == 1 and out.dtype == torch.int32
        assert words.dtype == torch.int32 and words.is_contiguous() and words.shape == (logits.shape[0], 4)
        self._run("sample", logits.numel() * 4, 0, None,
                  self.lib.llmrs_sample_rows, self._stream(), _p(logits), logits.stride(0), logits.shape[0],
                  logits.shape[1], _p(words), _p(out))


_kernels = None


def kernels():
    global _kernels
    if _kernels is None:
        _kernels = HipKernels()
    return _kernels


def stand_in_kernels() -> bool:
    """Whether another object stands in for the kernel library (`use_kernels`: tests of the host logic without a GPU)."""
    return _kernels is not None and not isinstance(_kernels, HipKernels)


@contextlib.contextmanager
def use_kernels(obj):
    """For tests: run the engine's host logic against a stand-in for the device."""
    global _kernels
    old, _kernels = _kernels, obj
    try:
        yield obj
    finally:
        _kernels = old

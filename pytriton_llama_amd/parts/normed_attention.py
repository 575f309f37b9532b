"""Softmax attention with normed queries and keys, keys and values of different sizes, and,
optionally, several score maps a head that are combined by difference."""
from __future__ import annotations

import math
from typing import List, Optional

import torch

from .. import ops
from .attention import ALL_16, PORTIONS_16, PORTIONS_64
from .base import PagedSpec, PagedTensor, ParamSource, Part, PendingSum, as_tensor, place, register_part
from .linear import LINEAR_LIBRARIES, decode_copy, linear
from .rotary import banded_inv_freq, ramp_inv_freq


def pad_rows(rows: torch.Tensor, multiple: int = 8) -> torch.Tensor:
    """``rows`` with zero rows added so that their number is a multiple (rows of the product's
    result then stay 16-byte aligned in bfloat16)."""
    pad = -rows.shape[0] % multiple
    return rows if not pad else torch.cat([rows, rows.new_zeros((pad, rows.shape[1]))], dim=0)


@register_part("mixer", "normed_attention")
class NormedAttention(Part):
    """Causal softmax attention over the paged cache:

        q = W_q x + b_q [heads, maps, dim],  k = W_k x + b_k [kv_heads, maps, dim],
        v = W_v x + b_v [kv_heads, vdim]
        q, k <- RMS norm (``qk_norm`` "head": over the dim entries of every head and map, one weight
                [dim] for all; "whole": over all of q and over all of k before they are split into
                heads, weights of that size; None: no norm), then rotation of the first rot_dims
                entries of every head (entry i with i + rot_dims / 2) by position * frequency
        a_m = softmax_j<=i (q_m(i) . k_m(j) * scale) v(j)         one result a map, same values
                (``window``: over the keys with i - j < window only, the query's own and the
                window - 1 before it; pages that every later query has left behind are given back.
                ``keep_first``: and over the keys at positions below it, which stay where they
                are and are never given back. ``sink_name``: a vector of the checkpoint, one
                number a head; the softmax denominator of head h also holds exp(sink_h), a term
                without key and value that the scale does not touch)

    maps = 1: out = W_o concat_h a + b_o.
    maps = 2 (differential attention: the second map is subtracted so that what both maps give
    to keys of no interest cancels): with lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff (one number
    for the layer, from four vectors of the checkpoint), o = a_1 - lam a_2, divided by its root mean
    square over vdim (no weight), times (1 - diff).
    ``gated``: the concatenated heads times sigmoid(W_g x) before the output projection.

    The cache keeps the normed and rotated keys [kv_heads * maps, dim] and the values [kv_heads,
    vdim] of every token. ``own_kv`` False: the layer has no key and value tensors and reads the
    cache layer of another one (the run order hands it over, not writable); sizes and rotation
    are the owner's. Scores, softmax, norms, angles and lam are float32; the projection's result is
    taken in float32 so that bias and norm see it unrounded. Tensor names are parameters; biases
    are the projection's name with ".b" added. ``rot_scaling``: None, or the numbers of a
    frequency scaling: factor, original, fast, slow (a ramp between the entries that turn fast and
    slow, parts/rotary.py: ramp_inv_freq, with its factor on sine and cosine) or factor, original,
    low, high (by wavelength band, banded_inv_freq)."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int,
                 scale: Optional[float] = None, eps: float = 1e-6, qk_norm: Optional[str] = "head",
                 maps: int = 1, diff: float = 0.0, bias: bool = True, gated: bool = False,
                 rot_dims: int = 0, rot_base: float = 10000.0, rot_scaling: Optional[dict] = None,
                 own_kv: bool = True, window: Optional[int] = None, keep_first: int = 0,
                 sink_name: Optional[str] = None, q_name: str = "q", k_name: str = "k", v_name: str = "v",
                 g_name: str = "g", o_name: str = "o", lambda_names=("lq1", "lk1", "lq2", "lk2")):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if maps not in (1, 2):
            raise ValueError(f"one or two score maps a head, got {maps}")
        if gated and maps == 1:
            raise ValueError("the output gate is built for two maps a head (it is applied where the maps "
                             "are combined)")
        if qk_norm not in (None, "head", "whole"):
            raise ValueError(f"unknown query/key norm {qk_norm!r} (known: 'head', 'whole', None)")
        if rot_dims % 2 or not 0 <= rot_dims <= dim:
            raise ValueError(f"{rot_dims} rotating entries of {dim}: an even number, at most the head's size")
        if max(dim, vdim) > 640:
            raise ValueError(f"the attention kernels take head sizes up to 640, got {dim} and {vdim}")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.maps = int(dim), int(vdim), int(maps)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(dim)
        self.eps, self.diff = float(eps), float(diff)
        self.norm_mode = {None: ops.NORM_NONE, "head": ops.NORM_HEAD, "whole": ops.NORM_WHOLE}[qk_norm]
        self.bias, self.gated, self.own_kv = bool(bias), bool(gated), bool(own_kv)
        self.rot_dims = int(rot_dims)
        if window is not None and window <= 0:
            raise ValueError("a window holds at least the query's own position")
        self.window = int(window) if window else None
        if keep_first < 0 or (keep_first and not self.window):
            raise ValueError("first positions are kept beside a window, and their number is not negative")
        self.keep_first = int(keep_first)
        if sink_name and maps != 1:
            raise ValueError("a term of the denominator without a key is built for one score map a head")
        self.sink_name = sink_name or None
        self.sink = None
        self.mag = 1.0
        self.inv_freq_host = None
        if self.rot_dims:
            if rot_scaling and "low" in rot_scaling:
                self.inv_freq_host = banded_inv_freq(
                    rot_base, self.rot_dims, float(rot_scaling["factor"]), float(rot_scaling["low"]),
                    float(rot_scaling["high"]), float(rot_scaling["original"]))
            elif rot_scaling:
                self.inv_freq_host, self.mag = ramp_inv_freq(
                    rot_base, self.rot_dims, float(rot_scaling["factor"]), float(rot_scaling["original"]),
                    float(rot_scaling["fast"]), float(rot_scaling["slow"]))
            else:
                i = torch.arange(0, self.rot_dims // 2, dtype=torch.float64)
                self.inv_freq_host = (float(rot_base) ** (-2.0 * i / self.rot_dims)).to(torch.float32)
        self.names = dict(q=q_name, k=k_name, v=v_name, g=g_name, o=o_name)
        self.lambda_names = tuple(lambda_names)
        self.q_size = self.num_heads * self.maps * self.dim
        self.k_size = self.num_kv_heads * self.maps * self.dim
        self.v_size = self.num_kv_heads * self.vdim
        self.o_size = self.num_heads * self.vdim
        self.k_off = self.q_size if self.own_kv else -1
        self.v_off = self.q_size + self.k_size
        self.g_off = self.q_size + (self.k_size + self.v_size if self.own_kv else 0)
        self.proj = self.o = self.proj_blocked = self.o_blocked = None
        self.q_bias = self.k_bias = self.v_bias = self.o_bias = None
        self.q_weight = self.k_weight = self.inv_freq = None
        self.lam = 0.0
        self.force_decode_splits = 0        # tests set it to try other splits
        libs = ("attention", "prepare", "stream") + LINEAR_LIBRARIES
        if self.dim % 32 == 0 and self.vdim % 32 == 0 and max(self.dim, self.vdim) <= 128:
            libs += ("attention_prefill",)          # the matrix-core kernel for prompt portions
        self.kernel_libraries = libs

    def work_lists(self):
        return (ALL_16, PORTIONS_16, PORTIONS_64)

    def decode_splits(self, ctx, n_dec: int, device, matrix_cores: bool = False) -> int:
        """How many workgroups share one decoding sequence's keys: enough to fill the compute
        units about twice over (measured on MI355X at batch 1 to 64 behind 2,048 keys: beyond that the
        merging of a workgroup's key slots costs more than the shorter loops save), never finer
        than one turn of a workgroup. ``matrix_cores``: for the matrix-core form (a workgroup a kv
        head, 128 keys a turn; no splits once the batch brings 1.75 workgroups a compute unit)."""
        if self.force_decode_splits:
            return self.force_decode_splits
        span = max(ctx.ctx_lens[:n_dec])
        if self.window:
            span = min(span, self.window + self.keep_first)
        cus = ops.compute_units(device)
        if matrix_cores:
            base = max(1, n_dec * self.num_kv_heads)
            want = 1 if 4 * base >= 7 * cus else -(-2 * cus // base)
            return max(1, min(want, -(-span // 128), 64))
        lpk = 1
        while lpk * 16 < max(self.dim, self.vdim):
            lpk <<= 1
        turn = 2 * (256 // lpk)
        per_kv = self.num_heads // self.num_kv_heads
        base = max(1, n_dec * self.num_kv_heads * self.maps * (-(-per_kv // 4)))
        want = -(-2 * cus // base)
        return max(1, min(want, -(-span // turn), 64))

    def attend(self, a, q, cache, ctx, group) -> None:
        """Leading sequences of one token: the split-KV kernel (its matrix-core form where one
        map reads keys and values of one size that it takes); the rest: the matrix-core kernel in
        64-row blocks (bfloat16, sizes that are multiples of 32 up to 128) or the vector kernel in
        16-row blocks."""
        n_dec = ctx.num_decode_seqs if ops.attention_decode_kv_fits(self.dim, self.vdim) else 0
        window = self.window or 0
        extras = dict(keep_first=self.keep_first, sink=self.sink)
        # one map and keys as large as values: the matrix-core form of the split-KV kernel takes them
        mfma = (n_dec and self.maps == 1 and self.dim == self.vdim and q.stride(0) % 8 == 0
                and ops.attention_decode_mfma_fits(q.dtype, self.num_heads, self.num_kv_heads, self.dim,
                                                   cache.page_size))
        if mfma:
            ops.attention_decode(a, q, cache.k, cache.v, ctx.q_start, ctx.ctx_len, group.block_table, n_dec,
                                 self.scale, window, self.decode_splits(ctx, n_dec, q.device, True),
                                 matrix_cores=True, **extras)
        elif n_dec:
            ops.attention_decode_kv(a, q, cache.k, cache.v, ctx.q_start, ctx.ctx_len, group.block_table, n_dec,
                                    self.scale, self.maps, self.decode_splits(ctx, n_dec, q.device), window,
                                    **extras)
        if n_dec == ctx.num_seqs:
            return
        if n_dec == ctx.num_decode_seqs and ops.attention_prefill_mfma_kv_fits(
                q.dtype, self.num_kv_heads, self.maps, self.dim, self.vdim, cache.page_size):
            ws, wo = ctx.work[PORTIONS_64]
            # as many workgroups a head as the chip holds at once share the list of blocks
            held = ops.compute_units(q.device) * (3 if self.dim + self.vdim <= 128 else 2)
            t = max(1, held // (self.num_heads * self.maps))
            blocks = ws.numel()
            ops.attention_prefill_mfma_kv(a, q, cache.k, cache.v, ctx.q_start, ctx.ctx_len, group.block_table,
                                          ws, wo, self.scale, self.maps, blocks if blocks <= 2 * t else t,
                                          window, **extras)
            return
        ws, wo = ctx.work[PORTIONS_16 if n_dec else ALL_16]
        ops.attention_generic_kv(a, q, cache.k, cache.v, ctx.q_start, ctx.ctx_len, group.block_table,
                                 ws, wo, self.scale, self.maps, window, **extras)

    def cache_spec(self):
        if not self.own_kv:
            return None
        return PagedSpec((PagedTensor("k", (self.num_kv_heads * self.maps, self.dim), 1),
                          PagedTensor("v", (self.num_kv_heads, self.vdim), 1)), self.window,
                         self.keep_first)

    def _norm_sizes(self):
        if self.norm_mode == ops.NORM_WHOLE:
            return self.q_size, self.k_size
        return self.dim, self.dim

    def param_sources(self) -> List[ParamSource]:
        n, W = self.names, self.hidden_size
        small = ("normal", 0.0, 0.1)
        out = [ParamSource(n["q"], (self.q_size, W))]
        if self.bias:
            out.append(ParamSource(n["q"] + ".b", (self.q_size,), "vector", init=small))
        if self.own_kv:
            out.append(ParamSource(n["k"], (self.k_size, W)))
            out.append(ParamSource(n["v"], (self.v_size, W)))
            if self.bias:
                out.append(ParamSource(n["k"] + ".b", (self.k_size,), "vector", init=small))
                out.append(ParamSource(n["v"] + ".b", (self.v_size,), "vector", init=small))
        if self.norm_mode != ops.NORM_NONE:
            nq, nk = self._norm_sizes()
            out.append(ParamSource(n["q"] + ".norm", (nq,), "vector"))
            if self.own_kv:
                out.append(ParamSource(n["k"] + ".norm", (nk,), "vector"))
        if self.maps == 2:
            out += [ParamSource(x, (self.dim,), "vector", init=("normal", 0.0, 0.1)) for x in self.lambda_names]
        if self.gated:
            out.append(ParamSource(n["g"], (self.o_size, W)))
        if self.sink_name:
            out.append(ParamSource(self.sink_name, (self.num_heads,), "vector", init=("normal", 0.0, 1.0)))
        out.append(ParamSource(n["o"], (W, self.o_size)))
        if self.bias:
            out.append(ParamSource(n["o"] + ".b", (W,), "vector", init=small))
        return out

    def load(self, tensors, dtype, device) -> None:
        n = self.names
        rows = [tensors[n["q"]]]
        if self.own_kv:
            rows += [tensors[n["k"]], tensors[n["v"]]]
        if self.gated:
            rows.append(tensors[n["g"]])
        self.proj = place(pad_rows(torch.cat(rows, dim=0)), "matrix", dtype, device)
        self.o = place(tensors[n["o"]], "matrix", dtype, device)
        if self.bias:
            self.q_bias = place(tensors[n["q"] + ".b"], "vector", dtype, device)
            self.o_bias = place(tensors[n["o"] + ".b"], "vector", dtype, device)
            if self.own_kv:
                self.k_bias = place(tensors[n["k"] + ".b"], "vector", dtype, device)
                self.v_bias = place(tensors[n["v"] + ".b"], "vector", dtype, device)
        if self.norm_mode != ops.NORM_NONE:
            self.q_weight = place(tensors[n["q"] + ".norm"], "vector", dtype, device)
            if self.own_kv:
                self.k_weight = place(tensors[n["k"] + ".norm"], "vector", dtype, device)
        if self.maps == 2:
            lq1, lk1, lq2, lk2 = (tensors[x].to(torch.float32).cpu() for x in self.lambda_names)
            self.lam = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum())) + self.diff
        if self.inv_freq_host is not None:
            self.inv_freq = self.inv_freq_host.to(device)
        if self.sink_name:
            self.sink = place(tensors[self.sink_name], "vector", dtype, device)

    def make_decode_copies(self) -> int:
        self.proj_blocked, self.o_blocked = decode_copy(self.proj), decode_copy(self.o)
        return sum(t.numel() * t.element_size() for t in (self.proj_blocked, self.o_blocked)
                   if t is not None)

    def heads_output(self, x, ctx, cache) -> torch.Tensor:
        """The concatenated heads [T, heads * vdim] in the engine's dtype: what the output
        projection reads."""
        x = as_tensor(x)
        T = x.shape[0]
        H, G, M, Dk, Dv = self.num_heads, self.num_kv_heads, self.maps, self.dim, self.vdim
        group = ctx.groups[cache.group]
        p = linear(x, self.proj, out_dtype=torch.float32, blocked=self.proj_blocked)
        q = torch.empty((T, H * M, Dk), dtype=x.dtype, device=x.device)
        ops.qkv_prepare(q, p, 0, self.k_off, self.v_off, self.q_bias, self.k_bias, self.v_bias,
                        self.norm_mode, self.q_weight, self.k_weight, self.eps, self.rot_dims,
                        self.inv_freq, self.mag, ctx.positions,
                        group.slots if (cache.writable and self.own_kv) else None, cache.k, cache.v,
                        H * M, G * M, G, Dk, Dv, cache.page_size)
        plain = M == 1
        a = torch.empty((T, H * M, Dv), dtype=x.dtype if plain else torch.float32, device=x.device)
        self.attend(a, q, cache, ctx, group)
        if plain:
            return a.view(T, H * Dv)
        out = torch.empty((T, H * Dv), dtype=x.dtype, device=x.device)
        ops.head_norm_gate(out, a, 2, self.lam, None, False, 1.0 - self.diff,
                           p if self.gated else None, self.g_off,
                           ops.GATE_SIGMOID if self.gated else ops.GATE_NONE, self.eps)
        return out

    def forward(self, x, ctx, cache):
        heads = self.heads_output(x, ctx, cache)
        y = linear(heads, self.o, out_dtype=torch.float32, blocked=self.o_blocked)
        return PendingSum([(y, 1.0)], (self.o_bias, 1.0) if self.bias else None)

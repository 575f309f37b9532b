"""Attention over a compressed (latent) cache that all heads share."""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .attention import PagedAttention
from .base import PagedSpec, PagedTensor, ParamSource, Part, as_tensor, place, register_part
from .linear import LINEAR_LIBRARIES, decode_copy, linear
from .rotary import ramp_inv_freq


def paired_inv_freq(base: float, dims: int) -> torch.Tensor:
    """f_i = base^(-2i / dims), i < dims / 2, for rotations of neighbouring pairs (2i, 2i + 1)."""
    i = torch.arange(0, dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / dims)).to(torch.float32)


@register_part("mixer", "latent_attention")
class LatentAttention(Part):
    """Causal softmax attention whose cache holds, per token, one latent vector c [kv_rank]
    (a down-projection of the input, RMS-normed) and one rotated key part kr [rot_dim]; every
    head's keys and values are linear maps of c:

        q_h = [qn_h | qr_h] = W_q x            qn_h [dim], qr_h [rot_dim] (rotated)
        score_h(i, j) = (qn_h(i) . Uk_h c_j + qr_h(i) . kr_j) * scale,  j <= i
        out = W_o concat_h( sigmoid(w_g,h . x) * Uv_h sum_j p_h(i, j) c_j )

    The maps move to the query side (q'_h = [Uk_h^T qn_h | qr_h], values c_j), so the attention
    kernels read the cache as it lies: one kv head of size kv_rank + rot_dim whose keys and
    values are the same pages (csrc/latent.hip). The rotation turns neighbouring pairs of the
    first ``rot_dims`` entries of the rotated part by position * rot_base^(-2i / rot_dims).

    ``own_kv`` False: the layer has no down-projection and reads the cache layer another one
    fills (the model's run order hands it that layer, not writable); its kv_rank, rot_dim and
    rotation are the owner's. ``gated`` False: no output gate. Tensor names are parameters.

    ``q_rank``: the queries pass through a latent of their own, q = W_uq (rmsnorm(W_dq x) w_q)
    (tensors ``dq_name``, ``q_norm_name``, ``uq_name`` instead of ``q_name``). ``rot_layout``
    "half": entry i of the rotating entries turns with entry i + rot_dims / 2 instead of its
    neighbour. ``rot_scaling`` (factor, original, fast, slow): frequencies along a ramp with a
    factor on sine and cosine (parts/rotary.py: ramp_inv_freq). ``sink_name``: a vector of the
    checkpoint, one number a head; the softmax denominator of head h also holds exp(sink_h), a
    term without key and value that the scale does not touch."""

    def __init__(self, hidden_size: int, num_heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                 scale: float, rot_base: float, rot_dims: Optional[int] = None, eps: float = 1e-6,
                 own_kv: bool = True, gated: bool = True, q_rank: Optional[int] = None,
                 rot_layout: str = "pairs", rot_scaling: Optional[dict] = None,
                 sink_name: Optional[str] = None,
                 q_name: str = "q", dkv_name: str = "dkv", c_norm_name: str = "dkv.norm",
                 uk_name: str = "uk", uv_name: str = "uv", g_name: str = "g", o_name: str = "o",
                 dq_name: str = "dq", q_norm_name: str = "dq.norm", uq_name: str = "uq"):
        rot_dims = rot_dim if rot_dims is None else int(rot_dims)
        if rot_layout not in ("pairs", "half"):
            raise ValueError(f"unknown layout of the rotating entries {rot_layout!r} (known: 'pairs', 'half')")
        if q_rank is not None and q_rank <= 0:
            raise ValueError("the queries' latent has a positive size")
        if rot_dim % 2 or rot_dims % 2 or rot_dims > rot_dim:
            raise ValueError(f"rotated size {rot_dim} with {rot_dims} rotating entries: both must be even, "
                             "the second at most the first")
        if kv_rank + rot_dim > 640:
            raise ValueError(f"the attention kernels take kv_rank + rot_dim up to 640, got {kv_rank + rot_dim}")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.dim, self.rot_dim, self.vdim, self.kv_rank = int(dim), int(rot_dim), int(vdim), int(kv_rank)
        self.scale, self.eps = float(scale), float(eps)
        self.own_kv, self.gated = bool(own_kv), bool(gated)
        self.q_rank = int(q_rank) if q_rank else 0
        self.half_layout = rot_layout == "half"
        self.mag = 1.0
        self.inv_freq_host = None
        if rot_dims and rot_scaling:
            self.inv_freq_host, self.mag = ramp_inv_freq(
                rot_base, rot_dims, float(rot_scaling["factor"]), float(rot_scaling["original"]),
                float(rot_scaling["fast"]), float(rot_scaling["slow"]))
        elif rot_dims:
            self.inv_freq_host = paired_inv_freq(rot_base, rot_dims)
        self.inv_freq: Optional[torch.Tensor] = None
        self.sink_name = sink_name or None
        self.names = dict(q=q_name, dkv=dkv_name, c_norm=c_norm_name, uk=uk_name, uv=uv_name, g=g_name, o=o_name,
                          dq=dq_name, q_norm=q_norm_name, uq=uq_name)
        D = self.kv_rank + self.rot_dim
        # the attention itself: the engine's paged attention with one kv head of size D whose
        # keys and values are the same pool
        self.core = PagedAttention(hidden_size, num_heads, 1, D, position=None, scale=self.scale)
        self.q_size = self.num_heads * (self.dim + self.rot_dim)
        first = self.q_rank or self.q_size             # the first rows of the fused projection
        self.kv_off = first if self.own_kv else -1
        self.g_off = first + (D if self.own_kv else 0)
        self.proj: Optional[torch.Tensor] = None          # rows q (or its latent) | down-projection | gate
        self.uq: Optional[torch.Tensor] = None            # [q_size, q_rank], with a latent of the queries
        self.q_weight: Optional[torch.Tensor] = None
        self.ukT: Optional[torch.Tensor] = None           # [H, kv_rank, dim]
        self.uv: Optional[torch.Tensor] = None            # [H, vdim, kv_rank]
        self.o: Optional[torch.Tensor] = None
        self.c_weight: Optional[torch.Tensor] = None
        self.proj_blocked = self.o_blocked = None
        libs = ("latent", "norm") + tuple(self.core.kernel_libraries)
        self.kernel_libraries = tuple(dict.fromkeys(l for l in libs if l != "rope"))

    @property
    def force_decode_splits(self) -> int:
        return self.core.force_decode_splits

    @force_decode_splits.setter
    def force_decode_splits(self, n: int) -> None:
        self.core.force_decode_splits = n

    def work_lists(self):
        return self.core.work_lists()

    def cache_spec(self):
        """One tensor a token, [c | kr]; pages [1, page_size, kv_rank + rot_dim]. A layer
        without a down-projection keeps nothing of its own."""
        if not self.own_kv:
            return None
        return PagedSpec((PagedTensor("latent", (1, self.kv_rank + self.rot_dim), 1),), None)

    def param_sources(self) -> List[ParamSource]:
        n, H, W = self.names, self.num_heads, self.hidden_size
        if self.q_rank:
            out = [ParamSource(n["dq"], (self.q_rank, W)), ParamSource(n["q_norm"], (self.q_rank,), "vector"),
                   ParamSource(n["uq"], (self.q_size, self.q_rank))]
        else:
            out = [ParamSource(n["q"], (self.q_size, W))]
        if self.own_kv:
            out += [ParamSource(n["dkv"], (self.kv_rank + self.rot_dim, W)),
                    ParamSource(n["c_norm"], (self.kv_rank,), "vector")]
        out += [ParamSource(n["uk"], (H * self.dim, self.kv_rank)),
                ParamSource(n["uv"], (H * self.vdim, self.kv_rank))]
        if self.gated:
            out.append(ParamSource(n["g"], (H, W)))
        if self.sink_name:
            out.append(ParamSource(self.sink_name, (H,), "vector", init=("normal", 0.0, 1.0)))
        out.append(ParamSource(n["o"], (W, H * self.vdim)))
        return out

    def load(self, tensors, dtype, device) -> None:
        n, H = self.names, self.num_heads
        if self.q_rank:
            rows = [tensors[n["dq"]]]
            self.uq = place(tensors[n["uq"]], "matrix", dtype, device)
            self.q_weight = place(tensors[n["q_norm"]], "vector", dtype, device)
        else:
            rows = [tensors[n["q"]]]
        if self.sink_name:
            self.core.sink = place(tensors[self.sink_name], "vector", dtype, device)
        if self.own_kv:
            rows.append(tensors[n["dkv"]])
            self.c_weight = place(tensors[n["c_norm"]], "vector", dtype, device)
        if self.gated:
            rows.append(tensors[n["g"]])
        rows = torch.cat(rows, dim=0)
        pad = -rows.shape[0] % 8            # (rows of the result stay 16-byte aligned in bfloat16)
        if pad:
            rows = torch.cat([rows, rows.new_zeros((pad, rows.shape[1]))], dim=0)
        self.proj = place(rows, "matrix", dtype, device)
        uk = tensors[n["uk"]].view(H, self.dim, self.kv_rank)
        self.ukT = place(uk.transpose(1, 2), "matrix", dtype, device)
        self.uv = place(tensors[n["uv"]].view(H, self.vdim, self.kv_rank), "matrix", dtype, device)
        self.o = place(tensors[n["o"]], "matrix", dtype, device)
        if self.inv_freq_host is not None:
            self.inv_freq = self.inv_freq_host.to(device)

    def make_decode_copies(self) -> int:
        self.proj_blocked, self.o_blocked = decode_copy(self.proj), decode_copy(self.o)
        return sum(t.numel() * t.element_size() for t in (self.proj_blocked, self.o_blocked)
                   if t is not None)

    def forward(self, x, ctx, cache):
        x = as_tensor(x)
        T, H, R, dr = x.shape[0], self.num_heads, self.kv_rank, self.rot_dim
        D = R + dr
        group = ctx.groups[cache.group]
        pool = cache.tensors["latent"]
        p = linear(x, self.proj, blocked=self.proj_blocked)
        # the queries: columns of the fused projection, or a second product from their normed latent
        qp = p if not self.q_rank else linear(ops.rmsnorm_cols(p[:, :self.q_rank], self.q_weight, self.eps),
                                              self.uq)
        q = torch.empty((T, H, D), dtype=x.dtype, device=x.device)
        ops.latent_prepare(q, p, 0, self.kv_off, ctx.positions, self.inv_freq, self.c_weight, self.eps,
                           group.slots if (cache.writable and self.own_kv) else None, pool,
                           H, self.dim, dr, R, queries=qp, half_layout=self.half_layout, mag=self.mag)
        if self.dim:
            qn = qp[:, :self.q_size].view(T, H, self.dim + dr)[:, :, :self.dim]
            ops.gemm_heads_nt(q[:, :, :R], qn, self.ukT)
        else:                               # (queries without an unrotated part: only kr is matched)
            q[:, :, :R].zero_()
        lat = torch.empty((T, H, D), dtype=x.dtype, device=x.device)
        self.core.attend(lat, q, cache, ctx, group, k=pool, v=pool)
        out = torch.empty((T, H, self.vdim), dtype=x.dtype, device=x.device)
        gate = p[:, self.g_off:self.g_off + H] if self.gated else None
        ops.gemm_heads_nt(out, lat[:, :, :R], self.uv, gate)
        return linear(out.view(T, H * self.vdim), self.o, blocked=self.o_blocked)

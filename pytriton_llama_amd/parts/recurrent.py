"""Mixers that carry a matrix of fixed size from token to token (csrc/recurrent.hip), and two
mixers side by side."""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .base import ParamSource, Part, PendingSum, StateSpec, as_tensor, place, register_part
from .linear import LINEAR_LIBRARIES, decode_copy, linear
from .normed_attention import pad_rows


class _MatrixStateMixer(Part):
    """What the two mixers below share: one fused first projection whose result is taken in
    float32, a float32 state slot, a result normed head by head and gated before the output
    projection."""
    kernel_libraries = ("recurrent", "prepare", "stream") + LINEAR_LIBRARIES

    def state_floats(self) -> int:
        raise NotImplementedError

    def cache_spec(self):
        return StateSpec((self.state_floats(),), torch.float32)

    def make_decode_copies(self) -> int:
        self.proj_blocked, self.o_blocked = decode_copy(self.proj), decode_copy(self.o)
        return sum(t.numel() * t.element_size() for t in (self.proj_blocked, self.o_blocked)
                   if t is not None)

    def forward(self, x, ctx, cache):
        heads = self.heads_output(as_tensor(x), ctx, cache)
        return linear(heads, self.o, out_dtype=torch.float32, blocked=self.o_blocked)


@register_part("mixer", "matrix_memory")
class MatrixMemory(_MatrixStateMixer):
    """The matrix memory of the xLSTM (Beck et al., "xLSTM: Extended Long Short-Term Memory"), with
    gates whose pre-activations are capped: per head, with q = W_q x * dim^-1/2, k = W_k x, v = W_v x,

        i = cap tanh((w_i . x + b_i) / cap),  f = logsigmoid(cap tanh((w_f . x + b_f) / cap))
        m' = max(f + m, i)                                   (m starts at 0)
        S <- exp(f + m - m') S + exp(i - m') k v^T,  n <- the same with k alone
        o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)

    then each head's o divided by its root mean square, times a weight of all heads' size, times
    sigmoid(W_g x), then W_o. S, n and m live in the request's state slot in float32; gates,
    exponentials and the recurrence are float32."""

    def __init__(self, hidden_size: int, num_heads: int, dim: int, vdim: int, gate_cap: float, eps: float,
                 q_name: str = "q", k_name: str = "k", v_name: str = "v", i_name: str = "i", f_name: str = "f",
                 g_name: str = "g", o_name: str = "o", norm_name: str = "norm"):
        if dim > 256:
            raise ValueError(f"the recurrence kernels take key sizes up to 256, got {dim}")
        if gate_cap <= 0:
            raise ValueError("gate_cap must be positive")
        self.hidden_size, self.num_heads, self.dim, self.vdim = int(hidden_size), int(num_heads), int(dim), int(vdim)
        self.cap, self.eps = float(gate_cap), float(eps)
        self.names = dict(q=q_name, k=k_name, v=v_name, i=i_name, f=f_name, g=g_name, o=o_name, norm=norm_name)
        H, D, Dv = self.num_heads, self.dim, self.vdim
        self.k_off, self.v_off = H * D, 2 * H * D
        self.g_off = 2 * H * D + H * Dv
        self.i_off = self.g_off + H * Dv
        self.f_off = self.i_off + H
        self.proj = self.o = self.proj_blocked = self.o_blocked = None
        self.i_bias = self.f_bias = self.norm_weight = None

    def state_floats(self) -> int:
        return ops.recurrent_state_floats(self.num_heads, self.dim, self.vdim)

    def param_sources(self) -> List[ParamSource]:
        n, W, H, D, Dv = self.names, self.hidden_size, self.num_heads, self.dim, self.vdim
        return [ParamSource(n["q"], (H * D, W)), ParamSource(n["k"], (H * D, W)), ParamSource(n["v"], (H * Dv, W)),
                ParamSource(n["g"], (H * Dv, W)), ParamSource(n["o"], (W, H * Dv)),
                ParamSource(n["norm"], (H * Dv,), "vector"),
                ParamSource(n["i"], (H, W)), ParamSource(n["i"] + ".b", (H,), "vector", init=("normal", 0.0, 1.0)),
                ParamSource(n["f"], (H, W)), ParamSource(n["f"] + ".b", (H,), "vector", init=("normal", 3.0, 1.0))]

    def load(self, tensors, dtype, device) -> None:
        n = self.names
        rows = torch.cat([tensors[n[x]] for x in ("q", "k", "v", "g", "i", "f")], dim=0)
        self.proj = place(pad_rows(rows), "matrix", dtype, device)
        self.o = place(tensors[n["o"]], "matrix", dtype, device)
        self.i_bias = place(tensors[n["i"] + ".b"], "vector", dtype, device)
        self.f_bias = place(tensors[n["f"] + ".b"], "vector", dtype, device)
        self.norm_weight = place(tensors[n["norm"]], "vector", dtype, device)

    def heads_output(self, x, ctx, cache) -> torch.Tensor:
        T, H, D, Dv = x.shape[0], self.num_heads, self.dim, self.vdim
        p = linear(x, self.proj, out_dtype=torch.float32, blocked=self.proj_blocked)
        o = ops.memory_scan(p, 0, self.k_off, self.v_off, self.i_off, self.f_off, self.i_bias, self.f_bias,
                            self.cap, D ** -0.5, cache.state, ctx.q_start, ctx.state_slots, H, D, Dv,
                            ctx.max_q_len)
        out = torch.empty((T, H * Dv), dtype=x.dtype, device=x.device)
        ops.head_norm_gate(out, o, 1, 0.0, self.norm_weight, True, 1.0, p, self.g_off, ops.GATE_SIGMOID, self.eps)
        return out


@register_part("mixer", "gated_delta")
class GatedDeltaRule(_MatrixStateMixer):
    """The gated delta rule (Yang, Kautz, Hatamizadeh, "Gated Delta Networks: Improving Mamba2 with
    Delta Rule"): q, k [kv_heads, dim] and v [heads, vdim] each pass a short causal convolution over
    time ([channels, taps], the last tap is the current token's) and SiLU; q and k become unit
    vectors x / sqrt(sum(x^2) + 1e-6), q also times dim^-1/2; per head, with beta = sigmoid(w_b . x)
    and g = exp(-exp(A_log) softplus(w_a . x + dt_bias)):

        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q

    then each head's o divided by its root mean square, times a weight [vdim] shared by the heads,
    times silu(W_g x), then W_o. S and the last taps - 1 inputs of the convolutions live in the
    request's state slot in float32. Head h uses q/k head h / (heads / kv_heads)."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, taps: int,
                 eps: float, q_name: str = "q", k_name: str = "k", v_name: str = "v", b_name: str = "b",
                 a_name: str = "a", g_name: str = "g", o_name: str = "o", norm_name: str = "norm",
                 A_log_name: str = "A_log", dt_bias_name: str = "dt_bias", conv_suffix: str = ".conv"):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} q/k heads")
        if dim > 256:
            raise ValueError(f"the recurrence kernels take key sizes up to 256, got {dim}")
        if taps < 1:
            raise ValueError("a convolution has at least one tap")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim, self.taps, self.eps = int(dim), int(vdim), int(taps), float(eps)
        self.names = dict(q=q_name, k=k_name, v=v_name, b=b_name, a=a_name, g=g_name, o=o_name,
                          norm=norm_name, A_log=A_log_name, dt_bias=dt_bias_name)
        self.conv_suffix = conv_suffix
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.dim, self.vdim
        self.channels = 2 * G * D + H * Dv
        self.g_off = self.channels
        self.a_off = self.g_off + H * Dv
        self.b_off = self.a_off + H
        self.tail_off = ops.recurrent_state_floats(H, D, Dv)
        self.proj = self.o = self.proj_blocked = self.o_blocked = None
        self.conv_weight = self.A_log = self.dt_bias = self.norm_weight = None

    def state_floats(self) -> int:
        return self.tail_off + (self.taps - 1) * self.channels

    def param_sources(self) -> List[ParamSource]:
        n, W, H, G, D, Dv, c = (self.names, self.hidden_size, self.num_heads, self.num_kv_heads, self.dim,
                                self.vdim, self.conv_suffix)
        conv = ("normal", 0.0, 0.5)
        return [ParamSource(n["q"], (G * D, W)), ParamSource(n["q"] + c, (G * D, self.taps), "vector", init=conv),
                ParamSource(n["k"], (G * D, W)), ParamSource(n["k"] + c, (G * D, self.taps), "vector", init=conv),
                ParamSource(n["v"], (H * Dv, W)), ParamSource(n["v"] + c, (H * Dv, self.taps), "vector", init=conv),
                ParamSource(n["b"], (H, W)), ParamSource(n["A_log"], (H,), "vector", init=("uniform", -3.0, 0.5)),
                ParamSource(n["norm"], (Dv,), "vector"), ParamSource(n["a"], (H, W)),
                ParamSource(n["dt_bias"], (H,), "vector", init=("normal", 0.0, 1.0)),
                ParamSource(n["g"], (H * Dv, W)), ParamSource(n["o"], (W, H * Dv))]

    def load(self, tensors, dtype, device) -> None:
        n, c = self.names, self.conv_suffix
        rows = torch.cat([tensors[n[x]] for x in ("q", "k", "v", "g", "a", "b")], dim=0)
        self.proj = place(pad_rows(rows), "matrix", dtype, device)
        self.o = place(tensors[n["o"]], "matrix", dtype, device)
        self.conv_weight = place(torch.cat([tensors[n[x] + c] for x in ("q", "k", "v")], dim=0), "vector", dtype, device)
        self.A_log = place(tensors[n["A_log"]], "vector", dtype, device)
        self.dt_bias = place(tensors[n["dt_bias"]], "vector", dtype, device)
        self.norm_weight = place(tensors[n["norm"]], "vector", dtype, device)

    def heads_output(self, x, ctx, cache) -> torch.Tensor:
        T, H, G, D, Dv = x.shape[0], self.num_heads, self.num_kv_heads, self.dim, self.vdim
        p = linear(x, self.proj, out_dtype=torch.float32, blocked=self.proj_blocked)
        q, k, v = ops.conv_prepare(p, 0, self.conv_weight, cache.state, self.tail_off, ctx.q_start,
                                   ctx.state_slots, G, H, D, Dv, D ** -0.5)
        ops.conv_tail_update(p, 0, self.channels, self.taps, cache.state, self.tail_off, ctx.q_start,
                             ctx.state_slots)
        o = ops.delta_scan(q, k, v, p, self.a_off, self.b_off, self.A_log, self.dt_bias, cache.state,
                           ctx.q_start, ctx.state_slots, ctx.max_q_len)
        out = torch.empty((T, H * Dv), dtype=x.dtype, device=x.device)
        ops.head_norm_gate(out, o, 1, 0.0, self.norm_weight, False, 1.0, p, self.g_off, ops.GATE_SILU, self.eps)
        return out


@register_part("mixer", "selective_scan")
class SelectiveScan(Part):
    """The selective scan of Mamba (Gu, Dao: "Mamba: Linear-Time Sequence Modeling with Selective
    State Spaces"): W_in x = [u | z] (``inner`` channels each); u passes a short causal
    convolution over time ([inner, taps], the last tap is the current token's, with a bias) and
    SiLU; W_x u = [r | B | C] (dt_rank, state, state entries); per channel c, with
    dt = softplus(w_dt[c] . r + b_c) and A = -exp(A_log),

        S[c, n] <- exp(dt A[c, n]) S[c, n] + dt u_c B_n;    y_c = sum_n S[c, n] C_n + D_c u_c

    then y * silu(z) and W_o. S [inner, state] and the convolution's last taps - 1 inputs live in
    the request's state slot in float32; the convolution, step sizes, decays and the recurrence are
    float32 (the two first projections' results are taken in float32, W_dt is held in float32)."""
    kernel_libraries = ("selective", "recurrent") + LINEAR_LIBRARIES

    def __init__(self, hidden_size: int, inner: int, state: int, dt_rank: int, taps: int,
                 in_name: str = "in", conv_name: str = "conv", conv_bias_name: str = "conv.b", x_name: str = "x",
                 dt_name: str = "dt", dt_bias_name: str = "dt.b", A_log_name: str = "A_log", D_name: str = "D",
                 o_name: str = "o"):
        if state > 256:
            raise ValueError(f"the scan kernel takes up to 256 states a channel, got {state}")
        if taps < 1:
            raise ValueError("a convolution has at least one tap")
        self.hidden_size, self.inner, self.state = int(hidden_size), int(inner), int(state)
        self.dt_rank, self.taps = int(dt_rank), int(taps)
        self.names = dict(i=in_name, conv=conv_name, conv_b=conv_bias_name, x=x_name, dt=dt_name,
                          dt_b=dt_bias_name, A_log=A_log_name, D=D_name, o=o_name)
        self.tail_off = self.inner * self.state
        self.w_in = self.w_x = self.o = self.w_in_blocked = self.w_x_blocked = self.o_blocked = None
        self.conv_weight = self.conv_bias = self.w_dt = self.dt_bias = self.A_log = self.D = None

    def cache_spec(self):
        return StateSpec((ops.selective_state_floats(self.inner, self.state, self.taps),), torch.float32)

    def param_sources(self) -> List[ParamSource]:
        n, W, C, N, R = self.names, self.hidden_size, self.inner, self.state, self.dt_rank
        return [ParamSource(n["i"], (2 * C, W)),
                ParamSource(n["conv"], (C, self.taps), "vector", init=("normal", 0.0, 0.5)),
                ParamSource(n["conv_b"], (C,), "vector", init=("normal", 0.0, 0.1)),
                ParamSource(n["x"], (R + 2 * N, C)),
                ParamSource(n["dt"], (C, R), "vector", init=("normal", 0.0, R ** -0.5)),
                ParamSource(n["dt_b"], (C,), "vector", init=("uniform", -4.0, -1.0)),
                ParamSource(n["A_log"], (C, N), "vector", init=("uniform", -1.0, 1.5)),
                ParamSource(n["D"], (C,), "vector"),
                ParamSource(n["o"], (W, C))]

    def load(self, tensors, dtype, device) -> None:
        n = self.names
        self.w_in = place(tensors[n["i"]], "matrix", dtype, device)
        self.w_x = place(pad_rows(tensors[n["x"]]), "matrix", dtype, device)
        self.o = place(tensors[n["o"]], "matrix", dtype, device)
        for attr, key in (("conv_weight", "conv"), ("conv_bias", "conv_b"), ("w_dt", "dt"), ("dt_bias", "dt_b"),
                          ("A_log", "A_log"), ("D", "D")):
            setattr(self, attr, place(tensors[n[key]], "vector", dtype, device))

    def make_decode_copies(self) -> int:
        self.w_in_blocked, self.w_x_blocked, self.o_blocked = (decode_copy(self.w_in), decode_copy(self.w_x),
                                                               decode_copy(self.o))
        return sum(t.numel() * t.element_size() for t in (self.w_in_blocked, self.w_x_blocked, self.o_blocked)
                   if t is not None)

    def forward(self, x, ctx, cache):
        x = as_tensor(x)
        C, N, R = self.inner, self.state, self.dt_rank
        p = linear(x, self.w_in, out_dtype=torch.float32, blocked=self.w_in_blocked)
        u, u_lp = ops.selective_conv(p, 0, self.conv_weight, self.conv_bias, cache.state, self.tail_off,
                                     ctx.q_start, ctx.state_slots, ctx.max_q_len, x.dtype)
        if self.taps > 1:
            ops.conv_tail_update(p, 0, C, self.taps, cache.state, self.tail_off, ctx.q_start, ctx.state_slots)
        r = linear(u if u_lp is None else u_lp, self.w_x, out_dtype=torch.float32, blocked=self.w_x_blocked)
        y = ops.selective_scan(u, p, C, r, R, R, R + N, self.w_dt, self.dt_bias, self.A_log, self.D,
                               cache.state, ctx.q_start, ctx.state_slots, x.dtype, ctx.max_q_len)
        return linear(y, self.o, out_dtype=torch.float32, blocked=self.o_blocked)


@register_part("mixer", "parallel")
class ParallelMixers(Part):
    """Two mixers side by side on one input: left_scale * left(x) + right_scale * right(x). Each
    keeps a cache of its own kind: ``cache_spec`` is a pair, and the model's run order hands the
    mixer a pair of cache layers. The sum is not made here: it is handed on (parts.base.PendingSum)
    to whoever reads the result next."""

    def __init__(self, left: Part, right: Part, left_scale: float = 1.0, right_scale: float = 1.0):
        self.left, self.right = left, right
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.kernel_libraries = tuple(dict.fromkeys(tuple(left.kernel_libraries) + tuple(right.kernel_libraries)))

    def children(self):
        """Sub-parts by the prefix their tensors carry inside this mixer's."""
        return {"left.": self.left, "right.": self.right}

    def cache_spec(self):
        return (self.left.cache_spec() if hasattr(self.left, "cache_spec") else None,
                self.right.cache_spec() if hasattr(self.right, "cache_spec") else None)

    def work_lists(self):
        lists = ()
        for m in (self.left, self.right):
            if hasattr(m, "work_lists"):
                lists += tuple(m.work_lists())
        return tuple(dict.fromkeys(lists))

    @property
    def graph_capturable(self) -> bool:
        return all(getattr(m, "graph_capturable", True) for m in (self.left, self.right))

    def param_sources(self) -> List[ParamSource]:
        out = []
        for prefix, m in self.children().items():
            for s in m.param_sources():
                out.append(ParamSource(prefix + s.name, s.shape, s.kind, s.init))
        return out

    def load(self, tensors, dtype, device) -> None:
        for prefix, m in self.children().items():
            m.load({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}, dtype, device)

    def make_decode_copies(self) -> int:
        return sum(m.make_decode_copies() for m in (self.left, self.right) if hasattr(m, "make_decode_copies"))

    def forward(self, x, ctx, cache):
        x = as_tensor(x)
        if not isinstance(cache, tuple) or len(cache) != 2:
            raise RuntimeError("two mixers side by side need a pair of cache layers")
        terms, bias = [], None
        for m, c, scale in ((self.left, cache[0], self.left_scale), (self.right, cache[1], self.right_scale)):
            y = m.forward(x, ctx, c)
            if isinstance(y, PendingSum) and len(y.terms) == 1 and (y.bias is None or bias is None):
                terms.append((y.terms[0][0], y.terms[0][1] * scale))
                if y.bias is not None:
                    bias = (y.bias[0], y.bias[1] * scale)
            else:
                terms.append((as_tensor(y), scale))
        if terms[0][0].dtype != terms[1][0].dtype:
            terms = [(t.float(), s) for t, s in terms]
        return PendingSum(terms, bias)

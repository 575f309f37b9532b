"""A plain, slow implementation of the Matusun design: whole sequences, no cache, one function a
mechanism, float64 on the CPU. It shares no code with the package; the tests compare the engine
with it.

A model is (config dict, tensors dict name -> torch tensor). Notation: h [T, W] is a sublayer's
input, rows are positions 0..T-1 of one sequence.

The design: a list of layers, each with one of two mixers (softmax attention inside a sliding
window; the selective scan of Mamba) and a routed feed-forward or none, RMS norms in front of
the sublayers, several residual streams mixed by learned matrices (hyper-connections), a range
of layers that runs several times, the embedding table as the head.
"""
from __future__ import annotations

import math

import torch

# The dtype an engine rounds to where it stores a result between kernels; None: nothing is rounded.
ROUND_TO = None

# When a list: every routed feed-forward appends a bool tensor [T]: whether the choice between the
# last expert taken and the first one left out is a close call that rounding may turn and that
# matters. Rounding moves a score by a small share of itself, so the call is close when the gap
# between the two choice scores is below CLOSE_CALL times the sum of the two scores; it matters
# when the expert taken has more than a thousandth of the token's weight.
ROUTER_MARGINS = None
CLOSE_CALL = 0.1


def stored(x):
    return x if ROUND_TO is None else x.to(ROUND_TO).to(x.dtype)


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def lin(h, w):
    return h @ w.T


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ---- attention -------------------------------------------------------------------------------
def rotate_half(x, positions, dims, base):
    """x [T, heads, D]: entry i of the first ``dims`` turns with entry i + dims / 2 by the angle
    position * base^(-2 i / dims); the rest of a head passes."""
    if dims == 0:
        return x
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    a = positions.to(torch.float64)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def window_mask(T, size):
    """[T, T] bool: row i sees column j when 0 <= i - j < size (``size`` None: every j <= i)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    vis = j <= i
    if size is not None:
        vis = vis & (i - j < size)
    return vis


def attention(h, m, w, eps, positions):
    """Grouped-query softmax attention: q and k RMS-normed over the whole projection, rotated,
    scores times the configured scale, a sliding window."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms(lin(h, w["q"]), eps) * w["q.norm"]
    k = rms(lin(h, w["k"]), eps) * w["k.norm"]
    v = lin(h, w["v"])
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = stored(rotate_half(q.view(T, H, D), positions, int(rot["dims"]), rot["base"]))
    k = stored(rotate_half(k.view(T, G, D), positions, int(rot["dims"]), rot["base"]))
    v = stored(v.view(T, G, Dv))
    size = (m.get("mask") or {}).get("size")
    vis = window_mask(T, None if size is None else int(size))
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        p = torch.softmax(s.masked_fill(~vis, float("-inf")), dim=-1)
        out[:, head] = p @ v[:, g]
    return lin(stored(out.reshape(T, H * Dv)), w["o"])


# ---- the selective scan ----------------------------------------------------------------------
def causal_conv(x, taps_w, bias):
    """x [T, C]; taps_w [C, taps], the last column is the current token's; zeros before the start."""
    T, C = x.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + padded[j:j + T] * taps_w[:, j]
    return y + bias


def selective_scan(x, dt, A, B, C, D):
    """x, dt [T, inner]; A [inner, state]; B, C [T, state]; D [inner]. One state matrix, from zero."""
    T, inner = x.shape
    S = torch.zeros(inner, A.shape[1], dtype=x.dtype)
    y = torch.zeros_like(x)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + D * x[t]
    return y


def mamba1(h, m, w):
    inner, state, rank = int(m["inner"]), int(m["state"]), int(m["dt_rank"])
    xz = lin(h, w["in"])
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, w["conv"], w["conv.b"]))
    p = lin(stored(x), w["x"])
    dt, B, C = p[:, :rank], p[:, rank:rank + state], p[:, rank + state:]
    dt = softplus(lin(dt, w["dt"]) + w["dt.b"])
    y = selective_scan(x, dt, -torch.exp(w["A_log"]), B, C, w["D"])
    return lin(stored(y * silu(z)), w["o"])


# ---- the routed feed-forward -----------------------------------------------------------------
def relu2_mlp(h, up, down):
    return lin(stored(torch.relu(lin(h, up)) ** 2), down)


def route(h, router, correction, top, scale):
    """(chosen experts [T, top], their weights [T, top], scores [T, E])."""
    s = torch.softmax(lin(h, router), dim=-1)
    choice = s + correction
    idx = torch.topk(choice, top, dim=-1).indices
    picked = torch.gather(s, 1, idx)
    if ROUTER_MARGINS is not None:
        if s.shape[1] > top:
            order = torch.sort(choice, dim=-1, descending=True)
            last, nxt = order.indices[:, top - 1:top], order.indices[:, top:top + 1]
            gap = (order.values[:, top - 1] - order.values[:, top])
            s_last, s_next = torch.gather(s, 1, last)[:, 0], torch.gather(s, 1, nxt)[:, 0]
            ROUTER_MARGINS.append((gap < CLOSE_CALL * (s_last + s_next)) & (s_last > 1e-3 * picked.sum(-1)))
        else:
            ROUTER_MARGINS.append(torch.zeros(h.shape[0], dtype=torch.bool))
    return idx, picked / (picked.sum(-1, keepdim=True) + 1e-20) * scale, s


def routed_mlp(h, mlp, w):
    r = mlp["router"]
    E, ident = int(r["experts"]), int(r.get("identity", 0))
    idx, wgt, _ = route(h, w["router"], w["correction"], int(r["top"]), float(r["scale"]))
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, f in zip(idx[t].tolist(), wgt[t]):
            if e >= E:                      # one of the last ``identity`` router outputs
                y[t] += f * h[t]
            else:
                y[t] += f * relu2_mlp(h[t:t + 1], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    if mlp.get("shared"):
        y = y + relu2_mlp(h, w["shared.up"], w["shared.down"])
    return y


# ---- a layer, the model -------------------------------------------------------------------------
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def mixer(h, layer, w, eps, positions):
    if layer["type"] == "attention":
        return attention(h, layer["mixer"], w, eps, positions)
    if layer["type"] == "mamba1":
        return mamba1(h, layer["mixer"], w)
    raise ValueError(layer["type"])


def hyper_sublayer(streams, hc, norm_w, eps, f):
    """streams [s, T, W]: u = sum_s in[s] x_s; y = f(norm(u)); x_t <- sum_s mix[s, t] x_s + out[t] y."""
    u = torch.einsum("s,stw->tw", hc["in"], streams)
    y = f(stored(rms(u, eps) * norm_w))
    return torch.einsum("sr,stw->rtw", hc["mix"], streams) + hc["out"][:, None, None] * y[None]


def layer_forward(streams, layer, w, eps, positions, hyper):
    def mix(a):
        return mixer(a, layer, sub(w, "mix."), eps, positions)

    def ff(a):
        return routed_mlp(a, layer["mlp"], sub(w, "mlp."))
    if hyper:
        streams = hyper_sublayer(streams, sub(w, "hc1."), w["norm1"], eps, mix)
        if layer.get("mlp"):
            streams = hyper_sublayer(streams, sub(w, "hc2."), w["norm2"], eps, ff)
        return streams
    x = streams[0]
    x = x + mix(stored(rms(x, eps) * w["norm1"]))
    if layer.get("mlp"):
        x = x + ff(stored(rms(x, eps) * w["norm2"]))
    return x[None]


def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg, tensors, tokens, dtype=torch.float64, round_to=None, layer_outputs=None):
    """Logits [T, vocab] of one sequence. ``round_to``: round where an engine of that dtype stores
    a result between kernels. ``layer_outputs``: a list that receives the residual stream (the sum
    of the streams) after every layer run."""
    global ROUND_TO
    ROUND_TO = round_to
    try:
        w = {k: v.to(dtype) for k, v in tensors.items()}
        eps = float(cfg["norm"]["eps"])
        tokens = torch.as_tensor(tokens, dtype=torch.long)
        positions = torch.arange(tokens.numel())
        x = w["embed"][tokens]
        hyper = cfg.get("streams") is not None
        n_streams = int(cfg["streams"]) if hyper else 1
        streams = x[None].repeat(n_streams, 1, 1)
        for i in run_order(cfg):
            streams = layer_forward(streams, cfg["layers"][i], sub(w, f"l{i}."), eps, positions, hyper)
            if layer_outputs is not None:
                layer_outputs.append(streams.sum(0))
        x = streams.sum(0)
        return lin(stored(rms(x, eps) * w["final.norm"]), w["embed"])
    finally:
        ROUND_TO = None

"""A plain, slow implementation of the Senavik design: whole sequences, no cache, one function a
mechanism, float64 on the CPU. It shares no code with the package; the tests compare the engine
with it.

A model is (config dict, tensors dict name -> torch tensor). Notation: h [T, W] is a sublayer's
input, rows are positions 0..T-1 of one sequence.

The design: an embedding with a norm behind it, a list of pre-norm layers, each with one of two
mixers (grouped-query attention inside a sliding window that also keeps the sequence's first
tokens; attention over a latent that all heads share, with queries that pass through a latent
of their own) and a dense or routed feed-forward or none, norms whose weights are stored as
their distance from one, a softmax whose denominator holds one learned term a head that belongs
to no key, and a head matrix of its own.
"""
from __future__ import annotations

import math

import torch

# The dtype an engine rounds to where it stores a result between kernels; None: nothing is rounded.
ROUND_TO = None

# When a list: every routed feed-forward appends a bool tensor [T]: whether rounding may turn the
# choice of groups or of experts (the gap between the last taken and the first left out is below
# CLOSE_CALL times the size of the two).
ROUTER_MARGINS = None
CLOSE_CALL = 0.02


def stored(x):
    return x if ROUND_TO is None else x.to(ROUND_TO).to(x.dtype)


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """The layers' and the model's norm: the weight is stored around zero."""
    return rms(x, eps) * (1.0 + w)


def lin(h, w):
    return h @ w.T


def silu(z):
    return z * torch.sigmoid(z)


# ---- rotation --------------------------------------------------------------------------------
def plain_freqs(base, dims):
    i = torch.arange(dims // 2, dtype=torch.float64)
    return float(base) ** (-2.0 * i / dims)


def banded_freqs(base, dims, scaling):
    """Frequencies rescaled by wavelength band (as Llama 3.1 does): waves shorter than
    original / high stay, waves longer than original / low are slowed by ``factor``, those between
    are blended. Returns (frequencies, factor on sine and cosine = 1)."""
    f = plain_freqs(base, dims)
    if not scaling:
        return f, 1.0
    factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
    original = float(scaling["original"])
    out = f.clone()
    for i in range(f.numel()):
        wave = 2.0 * math.pi / float(f[i])
        if wave < original / high:
            continue
        if wave > original / low:
            out[i] = f[i] / factor
        else:
            s = (original / wave - low) / (high - low)
            out[i] = (1.0 - s) * f[i] / factor + s * f[i]
    return out, 1.0


def ramped_freqs(base, dims, scaling):
    """Frequencies that go from f_i (entries that turn fast) to f_i / factor (slow ones) along a
    linear ramp, and the factor 0.1 ln(factor) + 1 on sine and cosine."""
    f = plain_freqs(base, dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def entry(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(entry(float(scaling["fast"]))), 0)
    hi = min(math.ceil(entry(float(scaling["slow"]))), dims - 1)
    out = f.clone()
    for i in range(f.numel()):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
    return out, 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, dims, freqs, mag=1.0):
    """x [T, heads, D]: entry i of the first ``dims`` turns with entry i + dims / 2 by the angle
    position * freqs[i], sine and cosine times ``mag``; the rest of a head passes."""
    if dims == 0:
        return x
    half = dims // 2
    a = positions.to(torch.float64)[:, None] * freqs[None, :]
    c, s = (torch.cos(a) * mag)[:, None, :].to(x.dtype), (torch.sin(a) * mag)[:, None, :].to(x.dtype)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# ---- what a query sees, and the softmax ------------------------------------------------------------
def visible(T, size=None, keep_first=0):
    """[T, T] bool: row i sees column j when j <= i and (i - j < size or j < keep_first);
    ``size`` None: every j <= i."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    vis = j <= i
    if size is not None:
        vis = vis & ((i - j < size) | (j < keep_first))
    return vis


def sink_softmax(s, vis, sink):
    """Softmax over the visible columns of s [T, T] whose denominator holds exp(sink) once more:
    a term without key and value (None: an ordinary softmax)."""
    s = s.masked_fill(~vis, float("-inf"))
    if sink is None:
        return torch.softmax(s, dim=-1)
    m = torch.maximum(s.max(dim=-1, keepdim=True).values, torch.as_tensor(sink, dtype=s.dtype))
    e = torch.exp(s - m)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - m))


# ---- the mixers ----------------------------------------------------------------------------------
def attention(h, m, w, positions):
    """Grouped-query attention, rotated on the first rot.dims entries of a head, inside a sliding
    window that keeps the first tokens, with a sink."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q, k, v = lin(h, w["q"]).view(T, H, D), lin(h, w["k"]).view(T, G, D), lin(h, w["v"]).view(T, G, Dv)
    rot = m.get("rot")
    if rot:
        f, mag = banded_freqs(rot["base"], int(rot["dims"]), rot.get("scaling"))
        q = rotate_half(q, positions, int(rot["dims"]), f, mag)
        k = rotate_half(k, positions, int(rot["dims"]), f, mag)
    q, k, v = stored(q), stored(k), stored(v)
    mask = m.get("mask")
    vis = visible(T) if not mask else visible(T, int(mask["size"]), int(mask.get("keep_first") or 0))
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * float(m["scale"])
        p = sink_softmax(s, vis, w["sink"][head] if "sink" in w else None)
        out[:, head] = p @ v[:, g]
    return lin(stored(out.reshape(T, H * Dv)), w["o"])


def latent_attention(h, m, w, eps, positions):
    """Attention whose keys and values are maps of one latent a token; queries pass through a
    latent too. All heads share one rotated key part."""
    T = h.shape[0]
    H, D, R, Dv, C = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    cq = stored(rms(lin(h, w["dq"]), eps) * w["dq.norm"])
    q = lin(cq, w["uq"]).view(T, H, D + R)
    down = lin(h, w["dkv"])
    c = stored(rms(down[:, :C], eps) * w["dkv.norm"])
    kr = down[:, C:].view(T, 1, R)
    rot = m["rot"]
    f, mag = ramped_freqs(rot["base"], int(rot["dims"]), rot.get("scaling"))
    qr = stored(rotate_half(q[:, :, D:], positions, int(rot["dims"]), f, mag))
    kr = stored(rotate_half(kr, positions, int(rot["dims"]), f, mag))[:, 0]
    qn = q[:, :, :D]
    kn = lin(c, w["uk"]).view(T, H, D)
    v = lin(c, w["uv"]).view(T, H, Dv)
    vis = visible(T)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for head in range(H):
        s = (qn[:, head] @ kn[:, head].T + qr[:, head] @ kr.T) * float(m["scale"])
        p = sink_softmax(s, vis, w["sink"][head] if "sink" in w else None)
        out[:, head] = p @ v[:, head]
    return lin(stored(out.reshape(T, H * Dv)), w["o"])


# ---- the feed-forwards -----------------------------------------------------------------------------
def dense_ff(h, w):
    """down(relu(up h)^2)."""
    return lin(stored(torch.relu(lin(h, w["up"])) ** 2), w["down"])


def route(h, mlp, w):
    """Which experts a token uses and with which weights: (indices [T, top], weights [T, top]).
    Scores are sigmoid(router h); the choice is by score + correction among the experts of the
    ``keep`` groups whose two best choice scores sum highest; the weights are the plain scores of
    the chosen, divided by their sum."""
    r = mlp["router"]
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(lin(h, w["router"]))
    choice = s + w["correction"]
    groups = r.get("groups")
    close = torch.zeros(h.shape[0], dtype=torch.bool)
    allowed = choice
    if groups:
        n, keep = int(groups["count"]), int(groups["keep"])
        per = E // n
        by_group = choice.view(-1, n, per)
        gs = by_group.topk(min(2, per), dim=-1).values.sum(-1)            # [T, n]
        order = gs.sort(dim=-1, descending=True, stable=True)
        best = order.indices[:, :keep]
        ok = torch.zeros_like(gs, dtype=torch.bool).scatter_(1, best, True)
        allowed = choice.masked_fill(~ok[:, :, None].expand(-1, -1, per).reshape(-1, E), float("-inf"))
        if keep < n:
            a, b = order.values[:, keep - 1], order.values[:, keep]
            close |= (a - b) < CLOSE_CALL * (a.abs() + b.abs())
    order = allowed.sort(dim=-1, descending=True, stable=True)
    idx = order.indices[:, :top]
    if top < E:
        a, b = order.values[:, top - 1], order.values[:, top]
        close |= torch.isfinite(b) & ((a - b) < CLOSE_CALL * (a.abs() + b.abs()))
    if ROUTER_MARGINS is not None:
        ROUTER_MARGINS.append(close)
    chosen = s.gather(1, idx)
    return idx, chosen / (chosen.sum(-1, keepdim=True) + 1e-20)


def expert(h, w, prefix):
    """down(silu(gate h) * (up h))."""
    return lin(stored(silu(lin(h, w[prefix + "gate"])) * lin(h, w[prefix + "up"])), w[prefix + "down"])


def routed_ff(h, mlp, w):
    idx, weights = route(h, mlp, w)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), weights[t]):
            out[t] += a * expert(h[t:t + 1], w, f"e{e}.")[0]
    return out


# ---- the model ---------------------------------------------------------------------------------------
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens, round_to=None, dtype=torch.float64, layers_out=None):
    """Logits [T, vocab] of one whole sequence. ``round_to``: the dtype an engine stores its
    intermediate results in (they are rounded to it where an engine rounds). ``layers_out``: a
    list that receives the residual stream behind every layer."""
    global ROUND_TO
    ROUND_TO = round_to
    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = float(cfg["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.numel())
    x = offset_norm(t["embed"][tokens], t["embed.norm"], eps)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = stored(offset_norm(x, t[p + "norm1"], eps))
        w = sub(t, p + "mix.")
        if layer["type"] == "attention":
            x = x + attention(h, layer["mixer"], w, positions)
        elif layer["type"] == "latent_attention":
            x = x + latent_attention(h, layer["mixer"], w, eps, positions)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = stored(offset_norm(x, t[p + "norm2"], eps))
            w = sub(t, p + "mlp.")
            x = x + (dense_ff(h, w) if mlp["kind"] == "dense" else routed_ff(h, mlp, w))
        if layers_out is not None:
            layers_out.append(x.clone())
    return lin(stored(offset_norm(x, t["final.norm"], eps)), t["head"])

"""Small Matusun configurations for the tests, none of them anyone's model. Between them they vary
every size and every branch: both mixers first and last, with and without a window, a rotation of
a whole head, of a part of it and none, one to four heads a kv head, key and value sizes that are
equal, that differ either way and that are no multiple of 16, sizes the matrix-core and split-KV
kernels take, 8 to 40 states a channel, channels that are no multiple of 16, one to four taps,
routed feed-forwards with and without experts that return their input, with and without a shared
expert, a token that takes every router output, layers without a feed-forward, one to five
residual streams and none (a plain residual sum), a looped range at the start, in the middle,
over all layers, run once, and none."""
import copy


def attention(heads, kv_heads, dim, vdim, scale, window=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    return "attention", m


def mamba(inner, state, dt_rank, conv):
    return "mamba1", {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def moe(ff, experts, top, scale, identity=None, shared=None):
    r = {"experts": experts, "top": top, "scale": scale}
    if identity is not None:
        r["identity"] = identity
    m = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def layer(kind_mixer, mlp):
    kind, m = kind_mixer
    return {"type": kind, "mixer": m, "mlp": mlp}


def model(vocab, width, eps, layers, streams=None, loop=None):
    cfg = {"architecture": "Matusun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams is not None:
        cfg["streams"] = streams
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def _m1():
    """Three streams; the middle two layers run twice; a window of 20 over pages of 4; a rotation of
    half a head; channels and states that fill their lanes unevenly; two experts that return their
    input."""
    a = attention(4, 2, 16, 24, 0.3, window=20, rot=(10000.0, 8))
    return model(200, 64, 1e-5, [
        layer(a, moe(40, 5, 2, 1.5, identity=2, shared=48)),
        layer(mamba(40, 8, 3, 4), moe(32, 4, 2, 0.8, identity=1)),
        layer(a, None),
        layer(mamba(72, 24, 5, 3), moe(40, 5, 3, 1.0, identity=2, shared=56)),
    ], streams=3, loop=(1, 3, 2))


def _m2():
    """No streams entry (a plain residual sum), no loop, the scan first and last, attention
    without a window and without a rotation, no experts that return their input and no shared
    expert, a layer without a feed-forward, a convolution of one tap (no inputs kept), 20 states,
    50 channels, one head a kv head, sizes that are no multiple of 16."""
    return model(150, 72, 1e-6, [
        layer(mamba(50, 20, 4, 1), moe(36, 3, 1, 2.0)),
        layer(attention(3, 3, 12, 20, 0.25), None),
        layer(attention(6, 2, 20, 12, 0.2, window=7, rot=(500.0, 20)), moe(24, 6, 2, 1.0, identity=0, shared=40)),
        layer(mamba(96, 40, 6, 2), None),
    ])


def _m3():
    """Sizes the matrix-core kernel for prompt portions and the split-KV decode kernel take (keys of
    32, values of 64, and the other way round), a window of 33 over pages of 16, one learned
    stream, all layers run twice, 16 states, a token takes every router output (3 of 2 + 1)."""
    return model(180, 96, 1e-5, [
        layer(attention(4, 2, 32, 64, 0.2, window=33, rot=(10000.0, 32)), moe(64, 2, 3, 1.2, identity=1, shared=64)),
        layer(mamba(128, 16, 8, 4), moe(64, 8, 2, 1.0, identity=2)),
        layer(attention(4, 4, 64, 32, 0.15, rot=(2000.0, 16)), None),
    ], streams=1, loop=(0, 3, 2))


def _m4():
    """Attention layers only (windows of 48 and 24 over pages of 8, and one without): what a key
    does to the logits is the attention's doing alone. Two streams; the first two layers run three
    times."""
    return model(200, 64, 1e-5, [
        layer(attention(4, 2, 32, 32, 0.18, window=48, rot=(10000.0, 32)), moe(48, 4, 2, 1.0, identity=1, shared=32)),
        layer(attention(2, 1, 16, 48, 0.25, window=24, rot=(800.0, 8)), None),
        layer(attention(4, 4, 32, 32, 0.18, rot=(10000.0, 16)), moe(48, 4, 1, 1.5)),
    ], streams=2, loop=(0, 2, 3))


def _m5():
    """Five streams, a loop that is run once, a window of one (a query sees itself alone), a
    window longer than any test sequence, the scan with four taps on 16 channels."""
    return model(120, 48, 1e-4, [
        layer(attention(2, 1, 8, 8, 0.35, window=1), moe(24, 3, 2, 1.0, identity=3)),
        layer(mamba(16, 12, 2, 4), None),
        layer(attention(3, 1, 24, 40, 0.2, window=4000, rot=(10000.0, 24)), moe(24, 3, 2, 1.0, shared=24)),
    ], streams=5, loop=(2, 3, 1))


# name -> (config, weight std, page size)
MATUSUN = {"M1": (_m1(), 0.12, 4), "M2": (_m2(), 0.15, 8), "M3": (_m3(), 0.12, 16), "M4": (_m4(), 0.12, 8),
           "M5": (_m5(), 0.15, 4)}


def matusun(name):
    cfg, std, page = MATUSUN[name]
    return copy.deepcopy(cfg), std, page

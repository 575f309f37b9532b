"""Small Senavik configurations for the tests, none of them anyone's model. Between them they vary
every size and every branch: both mixers first and last; windows of 1, shorter and longer than a
page, longer than any test sequence, and none; 0 to 17 kept first tokens (none, fewer than a page,
exactly a page, more than a page, more than the window); rotations of a whole head, of a part and
none, with and without rescaled frequencies, with band edges and ramps that meet all their
branches (also a ramp whose ends coincide); one to four heads a kv head; key and value sizes that
are equal, that differ either way and that are no multiple of 16; latents whose size with the
rotated part is 24, 32, 40, 64, 96 and 128 under 1 to 20 heads (so the vector, split-KV and
matrix-core kernels are all met); query latents smaller and larger than the width; dense, routed and absent feed-forwards;
experts in 1 to 6 groups of 1 to 4 of which 1 to all are kept, and no groups entry; 1 to 3
experts a token."""
import copy


def attention(heads, kv_heads, dim, vdim, scale, window=None, keep_first=None, rot=None, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
        if keep_first is not None:
            m["mask"]["keep_first"] = keep_first
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
        if scaling is not None:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return "attention", m


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot, scaling=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale, "rot": {"base": rot[0], "dims": rot[1]}}
    if scaling is not None:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return "latent_attention", m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, groups=None):
    r = {"experts": experts, "top": top}
    if groups is not None:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


def layer(kind_mixer, mlp):
    kind, m = kind_mixer
    return {"type": kind, "mixer": m, "mlp": mlp}


def model(vocab, width, eps, layers):
    return {"architecture": "Senavik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def _s1():
    """Pages of 4. A window of 20 that keeps 3 tokens (less than a page); frequencies in all three
    bands; a latent of 20 + 12 = 32 (the matrix-core kernels) with a ramp of two branches; eight
    experts in four pairs of which two are kept; a layer without a feed-forward."""
    a = attention(4, 2, 16, 24, 0.3, window=20, keep_first=3, rot=(10000.0, 8), scaling=(4.0, 1.0, 4.0, 64))
    l = latent(3, 8, 12, 12, 20, 16, 0.25, rot=(5000.0, 12), scaling=(4.0, 32, 8.0, 1.0))
    return model(200, 64, 1e-5, [
        layer(a, moe(40, 8, 2, groups=(4, 2))),
        layer(l, dense(48)),
        layer(a, None),
        layer(l, moe(32, 6, 3, groups=(3, 2))),
    ])


def _s2():
    """Pages of 8. The latent mixer first and last; attention without a window, and without a
    rotation; a window without kept tokens; no groups entry; one expert a token; sizes that are
    no multiple of 16 (latent 18 + 6 = 24: the vector kernel alone); a rotation of part of the
    rotated entries; a query latent larger than the width; a ramp whose ends coincide."""
    return model(150, 72, 1e-6, [
        layer(latent(2, 10, 6, 14, 18, 80, 0.3, rot=(800.0, 4), scaling=(8.0, 32, 64.0, 16.0)), moe(36, 3, 1)),
        layer(attention(3, 3, 12, 20, 0.25), None),
        layer(attention(6, 2, 20, 12, 0.2, window=7, rot=(500.0, 20)), moe(24, 6, 2, groups=(1, 1))),
        layer(latent(5, 6, 8, 8, 32, 24, 0.35, rot=(10000.0, 8)), dense(40)),
    ])


def _s3():
    """Pages of 16. Sizes the matrix-core and split-KV kernels take: keys of 32 with values of 64,
    keys and values of 64 with two heads a kv head; windows of 33 and 40 that keep 17 (more than a
    page) and 16 (a page); a latent of 48 + 16 = 64; six experts in three pairs, two pairs kept,
    three experts a token."""
    return model(180, 96, 1e-5, [
        layer(attention(4, 2, 32, 64, 0.2, window=33, keep_first=17, rot=(10000.0, 32), scaling=(8.0, 1.0, 4.0, 128)),
              moe(64, 6, 3, groups=(3, 2))),
        layer(latent(4, 16, 16, 32, 48, 40, 0.2, rot=(20000.0, 16), scaling=(2.0, 64, 16.0, 2.0)), dense(64)),
        layer(attention(4, 2, 64, 64, 0.15, window=40, keep_first=16, rot=(2000.0, 16)), moe(48, 4, 2, groups=(2, 1))),
        layer(latent(2, 32, 32, 64, 64, 32, 0.15, rot=(10000.0, 32)), None),
    ])


def _s4():
    """Attention layers only (windows of 48 and 24 over pages of 8 that keep 5 and 8 tokens, and
    one without a window): what a key does to the logits is the attention's doing alone."""
    return model(200, 64, 1e-5, [
        layer(attention(4, 2, 32, 32, 0.18, window=48, keep_first=5, rot=(10000.0, 32)), dense(48)),
        layer(attention(2, 1, 16, 48, 0.25, window=24, keep_first=8, rot=(800.0, 8), scaling=(4.0, 1.0, 2.0, 40)), None),
        layer(attention(4, 4, 32, 32, 0.18, rot=(10000.0, 16)), moe(48, 4, 1, groups=(4, 2))),
    ])


def _s5():
    """Pages of 4. A window of one (a query sees itself and the kept tokens), kept tokens beyond
    the window, a window longer than any test sequence, one head, four heads a kv head, groups of
    one expert, every group kept, a latent of 32 + 8 = 40 (split-KV and vector kernels)."""
    return model(120, 48, 1e-4, [
        layer(attention(2, 1, 8, 8, 0.35, window=1, keep_first=2), moe(24, 4, 2, groups=(4, 3))),
        layer(latent(1, 8, 8, 16, 32, 12, 0.3, rot=(10000.0, 8), scaling=(4.0, 16, 4.0, 1.0)), None),
        layer(attention(4, 1, 24, 40, 0.2, window=6, keep_first=9, rot=(10000.0, 24)), moe(24, 3, 2, groups=(3, 3))),
        layer(attention(1, 1, 16, 16, 0.3, window=4000, keep_first=4, rot=(100.0, 16)), dense(32)),
    ])


def _s6():
    """Pages of 16. Head sizes of real models: attention with keys and values of 128, four heads a kv
    head, half a head rotating, a window of 64 that keeps 4; latents of 96 + 32 = 128 under 16 heads
    (the most the matrix-core decode kernel takes on one kv head) and under 20 (the vector split-KV
    kernel); 16 experts in 4 groups of which 2 are kept."""
    return model(300, 128, 1e-6, [
        layer(attention(8, 2, 128, 128, 0.09, window=64, keep_first=4, rot=(500000.0, 64), scaling=(8.0, 1.0, 4.0, 256)),
              dense(160)),
        layer(latent(16, 64, 32, 64, 96, 96, 0.1, rot=(10000.0, 32), scaling=(40.0, 128, 32.0, 1.0)),
              moe(64, 16, 2, groups=(4, 2))),
        layer(latent(20, 32, 32, 32, 96, 48, 0.12, rot=(10000.0, 32)), None),
    ])


# name -> (config, weight std, page size)
SENAVIK = {"S1": (_s1(), 0.12, 4), "S2": (_s2(), 0.15, 8), "S3": (_s3(), 0.12, 16), "S4": (_s4(), 0.12, 8),
           "S5": (_s5(), 0.15, 4), "S6": (_s6(), 0.08, 16)}


def senavik(name):
    cfg, std, page = SENAVIK[name]
    return copy.deepcopy(cfg), std, page


def drawn(seed):
    """A configuration drawn from the ranges a model of this design may lie in (pages of 16):
    2 to 5 layers of either kind in any order, head sizes 16 to 128, 1 to 4 heads a kv head,
    windows from 8 to 130 or none with 0 to 20 kept tokens, rotations of none, part or all of a
    head with or without rescaled frequencies, latents of 40 to 128 with the rotated part, dense,
    routed or absent feed-forwards with 4 to 32 experts in groups."""
    import random
    rng = random.Random(seed)
    width = rng.choice([64, 96, 128, 192, 256])
    layers = []
    for _ in range(rng.randint(2, 5)):
        if rng.random() < 0.55:
            kv = rng.choice([1, 2, 4])
            dim, vdim = rng.choice([16, 32, 48, 64, 96, 128]), rng.choice([16, 32, 48, 64, 96, 128])
            if rng.random() < 0.5:
                vdim = dim
            window = rng.choice([None, 8, 33, 64, 96, 130])
            keep = rng.choice([None, 0, 1, 4, 16, 20]) if window else None
            rot = None
            if rng.random() < 0.85:
                rot = (rng.choice([10000.0, 20000.0, 500000.0]), rng.choice([dim, dim // 2, 8]))
            scaling = (rng.choice([2.0, 8.0]), 1.0, rng.choice([2.0, 4.0]), rng.choice([32, 64, 256])) \
                if rot and rng.random() < 0.7 else None
            mixer = attention(kv * rng.choice([1, 2, 4]), kv, dim, vdim, rng.uniform(0.7, 1.3) * dim ** -0.5,
                              window=window, keep_first=keep, rot=rot, scaling=scaling)
        else:
            dim, rot_dim = rng.choice([16, 32, 64]), rng.choice([8, 16, 32])
            kv_rank = rng.choice([32, 48, 64, 96])
            scaling = (rng.choice([4.0, 40.0]), rng.choice([32, 128]), rng.choice([8.0, 32.0]), rng.choice([1.0, 2.0])) \
                if rng.random() < 0.7 else None
            mixer = latent(rng.choice([2, 4, 6, 8, 16]), dim, rot_dim, rng.choice([16, 32, 64, 80]), kv_rank,
                           rng.choice([32, 64, 128]), rng.uniform(0.7, 1.3) * (dim + rot_dim) ** -0.5,
                           rot=(rng.choice([10000.0, 250000.0]), rot_dim), scaling=scaling)
        kind = rng.random()
        if kind < 0.2:
            mlp = None
        elif kind < 0.45:
            mlp = dense(rng.choice([64, 96, 256]))
        else:
            experts = rng.choice([4, 8, 16, 32])
            count = rng.choice([c for c in (1, 2, 4, 8) if experts % c == 0])
            keep_groups = rng.randint(1, count)
            top = rng.randint(1, min(4, keep_groups * (experts // count)))
            mlp = moe(rng.choice([32, 64, 96]), experts, top, groups=(count, keep_groups) if rng.random() < 0.85 else None)
            if mlp["router"].get("groups") is None:
                mlp = moe(mlp["expert"]["ff"], experts, min(top, experts))
        layers.append(layer(mixer, mlp))
    return model(rng.randint(100, 600), width, rng.choice([1e-6, 1e-5]), layers), 0.1, 16

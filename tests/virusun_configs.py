"""Small Virusun configurations for the tests, none of them anyone's model. Between them they vary
every size and every branch: the three mixers in every order (each of them first and last), layers
that read another's keys and values, layers without a feed-forward, key sizes and value sizes that
are equal, that differ either way and that are no multiple of 16, one to three heads a kv head,
rotations of a whole head and of a part of it, with and without the ramp between scaled and
unscaled frequencies, convolutions of one to four taps, more than 16 value columns a head block."""
import copy


def attention(heads, kv_heads, dim, vdim, scale, diff, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "attention", m


def parallel(left, right, left_scale, right_scale):
    return "parallel", {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def rotary(heads, kv_heads, dim, vdim, scale, base, dims, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}


def memory(heads, dim, vdim, gate_cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}


def delta(heads, kv_heads, dim, vdim, conv):
    return "delta", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def layer(kind_mixer, ff):
    kind, m = kind_mixer
    return {"type": kind, "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def model(vocab, width, eps, layers):
    return {"architecture": "Virusun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


def _v1():
    a = dict(heads=6, kv_heads=2, dim=16, vdim=24, scale=0.3, diff=0.4)
    return model(200, 64, 1e-5, [
        layer(attention(**a), 96),
        layer(delta(4, 2, 16, 24, 4), 80),
        layer(attention(**a, kv_from=0), None),
        layer(parallel(rotary(4, 2, 32, 16, 0.2, 10000.0, 32, (4.0, 64, 8.0, 1.0)), memory(3, 16, 24, 10.0), 0.8, 1.3), 72),
        layer(attention(**a), 64),
    ])


def _v2():
    """Starts with the delta rule, ends with two mixers side by side; sizes that are no multiple of 16;
    a rotation of a part of the head without the ramp; one head a kv head."""
    return model(150, 72, 1e-6, [
        layer(delta(3, 3, 20, 12, 2), None),
        layer(attention(3, 3, 12, 20, 0.25, 0.7), 100),
        layer(delta(2, 1, 40, 36, 3), 56),
        layer(parallel(rotary(3, 1, 24, 40, 0.15, 500.0, 12), memory(2, 24, 20, 4.0), 1.0, 0.5), None),
    ])


def _v3():
    """Starts with two mixers side by side; key size above value size in the differential layers; a
    convolution of one tap (no inputs kept); value sizes above 16 and 32 (several column blocks)."""
    a = dict(heads=4, kv_heads=4, dim=40, vdim=8, scale=0.2, diff=0.25)
    return model(120, 96, 1e-4, [
        layer(parallel(rotary(8, 4, 16, 16, 0.25, 2000.0, 8, (2.0, 32, 4.0, 0.5)), memory(1, 48, 40, 20.0), 1.5, 0.7), 64),
        layer(attention(**a), None),
        layer(delta(2, 2, 32, 48, 1), 48),
        layer(attention(**a, kv_from=1), 80),
        layer(attention(heads=2, kv_heads=1, dim=8, vdim=8, scale=0.35, diff=0.5, kv_from=None), 40),
        layer(delta(6, 2, 8, 8, 4), 40),
    ])


def _v4():
    """Attention layers only (differential ones, one that reads another's keys and values, and a
    rotary one whose neighbour is scaled to nothing): what a far key does to the logits is the
    attention's doing alone."""
    a = dict(heads=4, kv_heads=2, dim=32, vdim=32, scale=0.18, diff=0.3)
    return model(200, 64, 1e-5, [
        layer(attention(**a), 64),
        layer(parallel(rotary(4, 2, 32, 32, 0.18, 10000.0, 32, (8.0, 128, 16.0, 2.0)), memory(1, 8, 8, 5.0), 1.0, 0.0), 64),
        layer(attention(**a, kv_from=0), 64),
    ])


def _v5():
    """Sizes that the matrix-core kernel for prompt portions and the split-KV decode kernel take, with
    keys and values of different sizes either way (32 / 64 in the differential layers, 64 / 32 beside
    the matrix memory), two heads a kv head, a key size of 64 in the recurrences."""
    a = dict(heads=4, kv_heads=2, dim=32, vdim=64, scale=0.2, diff=0.35)
    return model(180, 96, 1e-5, [
        layer(parallel(rotary(4, 2, 64, 32, 0.15, 10000.0, 32, (4.0, 64, 8.0, 1.0)), memory(2, 64, 32, 12.0), 0.9, 1.1), 80),
        layer(attention(**a), 72),
        layer(delta(4, 2, 64, 32, 3), None),
        layer(attention(**a, kv_from=1), 64),
    ])


# name -> (config, weight std, page size)
VIRUSUN = {"V1": (_v1(), 0.12, 16), "V2": (_v2(), 0.15, 4), "V3": (_v3(), 0.12, 8), "V4": (_v4(), 0.12, 16),
           "V5": (_v5(), 0.12, 16)}


def virusun(name):
    cfg, std, page = VIRUSUN[name]
    return copy.deepcopy(cfg), std, page

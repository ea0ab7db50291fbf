"""Small Rubasun configurations for the tests, none of them anyone's model. Between them they
vary every size and every branch: layers with a cache of their own and layers that read
another's, dense, routed and absent feed-forwards, one or several experts a token, with and
without a shared expert, with and without the per-layer token input, rotated parts that turn
wholly or in part, latent sizes that the matrix-core attention takes (64), that only the
vector kernels take (48, 160) and that are no multiple of 16 (42), more than 16 heads."""
import copy


def mixer(heads, dim, rot_dim, vdim, kv_rank, scale, base, rot_dims=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit, shared_ff=None, shared_limit=None):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared_ff:
        m["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return m


def layer(m, mlp):
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def model(vocab, width, emb_scale, eps, side_dim, layers):
    cfg = {"architecture": "Rubasun", "vocab": vocab, "width": width, "embedding": {"scale": emb_scale},
           "norm": {"eps": eps}, "layers": layers}
    if side_dim:
        cfg["token_side"] = {"dim": side_dim}
    return cfg


def _r1():
    m = dict(heads=4, dim=16, rot_dim=16, vdim=24, kv_rank=48, scale=0.2, base=10000.0)
    return model(200, 64, 6.0, 1e-5, 8, [
        layer(mixer(**m), dense(96)),
        layer(mixer(**m), moe(5, 2, 40, 1.5, 56, 2.5)),
        layer(mixer(**m, kv_from=1), moe(5, 2, 40, 1.5)),
        layer(mixer(**m, kv_from=1), None),
        layer(mixer(**m), dense(72)),
    ])


def _r2():
    m = dict(heads=5, dim=24, rot_dim=8, vdim=16, kv_rank=40, scale=0.15, base=500.0)
    return model(300, 96, 1.0, 1e-6, 0, [
        layer(mixer(**m), moe(3, 1, 64, 3.0, 32, 1.0)),
        layer(mixer(**m, kv_from=0), dense(128)),
        layer(mixer(**m), moe(3, 3, 48, 2.0)),
    ])


def _r3():
    m = dict(heads=20, dim=8, rot_dim=32, vdim=8, kv_rank=128, scale=0.1, base=80000.0, rot_dims=16)
    return model(160, 128, 3.0, 1e-4, 4, [
        layer(mixer(**m), moe(8, 3, 32, 2.0, 64, 2.0)),
        layer(mixer(**m, kv_from=0), moe(8, 3, 32, 2.0, 64, 2.0)),
    ])


def _r4():
    m = dict(heads=3, dim=10, rot_dim=6, vdim=12, kv_rank=36, scale=0.25, base=100.0)
    return model(120, 72, 2.5, 1e-6, 5, [
        layer(mixer(**m), None),
        layer(mixer(**m, kv_from=0), dense(100)),
        layer(mixer(**m), moe(4, 2, 24, 1.0, 24, 1.0)),
    ])


def _r5():
    """Two cache shapes in one model (two page pools, two block tables a request), heads and
    sizes that change from layer to layer, a borrowed cache behind each."""
    a = dict(heads=2, dim=8, rot_dim=16, vdim=8, kv_rank=16, scale=0.3, base=1000.0)
    b = dict(heads=6, dim=16, rot_dim=8, vdim=16, kv_rank=56, scale=0.2, base=20000.0, rot_dims=4)
    a2 = dict(a, heads=4, dim=4, vdim=20)
    return model(90, 80, 4.0, 1e-5, 3, [
        layer(mixer(**a), dense(40)),
        layer(mixer(**b), moe(6, 2, 16, 2.0, 8, 2.0)),
        layer(mixer(**a2, kv_from=0), moe(6, 1, 16, 2.0)),
        layer(mixer(**b, kv_from=1), dense(64)),
    ])


def _r6():
    """A latent as wide as those of the largest public models of this kind (512 + 64): beyond
    the head sizes of the matrix-core and split-KV kernels, the vector kernel takes it."""
    m = dict(heads=2, dim=8, rot_dim=64, vdim=8, kv_rank=512, scale=0.1, base=10000.0)
    return model(100, 64, 2.0, 1e-6, 0, [layer(mixer(**m), dense(48)), layer(mixer(**m, kv_from=0), None)])


def _r7():
    """More than 16 heads on a latent size that the matrix-core kernels take (prompt portions on
    the matrix cores, decoded tokens through the vector split-KV kernel), one expert a token."""
    m = dict(heads=18, dim=8, rot_dim=32, vdim=8, kv_rank=64, scale=0.12, base=3000.0)
    return model(150, 96, 5.0, 1e-6, 2, [layer(mixer(**m), moe(7, 1, 24, 1.5, 16, 1.5)),
                                        layer(mixer(**m, kv_from=0), dense(80)),
                                        layer(mixer(**m), None)])


# name -> (config, weight std, page size)
RUBASUN = {"R1": (_r1(), 0.12, 16), "R2": (_r2(), 0.10, 4), "R3": (_r3(), 0.10, 8), "R4": (_r4(), 0.15, 16),
           "R5": (_r5(), 0.15, 8), "R6": (_r6(), 0.12, 16),
           "R7": (_r7(), 0.10, 16)}


def rubasun(name):
    cfg, std, page = RUBASUN[name]
    return copy.deepcopy(cfg), std, page

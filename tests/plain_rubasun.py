"""A plain, slow Rubasun: whole sequences, no cache, float32 (or float64) on the CPU.

One function per mechanism, written from the design's equations and sharing no code with the
engine. ``weights`` is a dict name -> tensor with the checkpoint's names; ``cfg`` is the
config.json dict. With ``round_to`` set to torch.bfloat16 the matrices are rounded as the engine
holds them (the arithmetic stays in the wide type).
"""
import math

import torch


def dyt(x, w, b, alpha):
    """Dynamic Tanh: tanh(alpha x) w + b, no statistics."""
    return torch.tanh(alpha * x) * w + b


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_pairs(x, positions, base, dims):
    """x [..., T, n]: the first ``dims`` entries in neighbouring pairs (2i, 2i+1), angle
    p * base^(-2i/dims); the rest unchanged."""
    out = x.clone()
    half = dims // 2
    f = base ** (-2.0 * torch.arange(half, dtype=x.dtype) / dims)
    a = positions.to(x.dtype)[:, None] * f[None, :]                 # [T, half]
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_kv(h, W, name, m, eps, positions):
    """The latent c [T, kv_rank] and the shared rotated key part [T, rot_dim] of a layer that
    owns a down projection."""
    r = m["kv_rank"]
    d = h @ W[name + ".mix.dkv"].T
    c = rms(d[:, :r], eps) * W[name + ".mix.dkv.norm"]
    kr = rotate_pairs(d[:, r:], positions, m["rot"]["base"], m["rot"]["dims"])
    return c, kr


def latent_attention(h, W, name, m, c, kr, positions):
    """Causal softmax attention with per-head keys and values expanded from the latent."""
    T = h.shape[0]
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    q = (h @ W[name + ".mix.q"].T).view(T, H, dn + dr)
    qn = q[..., :dn]
    qr = rotate_pairs(q[..., dn:].transpose(0, 1), positions, m["rot"]["base"], m["rot"]["dims"]).transpose(0, 1)
    kn = (c @ W[name + ".mix.uk"].T).view(T, H, dn)
    v = (c @ W[name + ".mix.uv"].T).view(T, H, dv)
    s = (torch.einsum("ihd,jhd->hij", qn, kn) + torch.einsum("ihd,jd->hij", qr, kr)) * m["scale"]
    i = torch.arange(T)
    s = s.masked_fill(i[None, :] > i[:, None], float("-inf"))
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhd->ihd", p, v)
    o = o * torch.sigmoid(h @ W[name + ".mix.g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ W[name + ".mix.o"].T


def dense_ff(h, W, prefix):
    g = h @ W[prefix + ".gate"].T
    return (g * torch.sigmoid(g) * (h @ W[prefix + ".up"].T)) @ W[prefix + ".down"].T


def clamped_expert(h, W, prefix, limit):
    g = torch.clamp(h @ W[prefix + ".gate"].T, max=limit)
    u = torch.clamp(h @ W[prefix + ".up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ W[prefix + ".down"].T


def moe_ff(h, W, prefix, mlp, margins_out=None):
    """``margins_out``: a list that receives, per token, by how much the logit of its last
    chosen expert exceeds that of the best expert left out (inf when all are chosen)."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ W[prefix + ".router"].T                                 # [T, E]
    s = torch.sigmoid(z)
    val, idx = torch.topk(s, top, dim=-1)
    if margins_out is not None:
        zs = z.sort(-1, descending=True).values
        margins_out.append(zs[:, top - 1] - zs[:, top] if top < E else torch.full_like(zs[:, 0], float("inf")))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(top):
            e = int(idx[t, k])
            out[t] += clamped_expert(val[t, k] * h[t:t + 1], W, f"{prefix}.e{e}", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        sg = torch.sigmoid(h @ W[prefix + ".shared.sg"].T)          # [T, 1]
        out = out + sg * clamped_expert(h, W, prefix + ".shared", mlp["shared"]["limit"])
    return out


def token_side(x, tokens, W, name, layer, dim, eps):
    e = W["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(x @ W[name + ".side.gate"].T) * e
    y = g @ W[name + ".side.proj"].T
    return x + rms(y, eps) * W[name + ".side.norm"]


def norm_of(x, W, name):
    return dyt(x, W[name], W[name + ".b"], W[name + ".alpha"])


def forward(cfg, weights, tokens, dtype=torch.float32, round_to=None, layers_out=None, margins_out=None):
    """Logits [T, vocab] of one whole sequence. ``layers_out``: a list that receives the
    residual stream after every layer; ``margins_out``: see moe_ff (one entry a routed layer)."""
    W = {}
    for k, t in weights.items():
        if t.dtype in (torch.int32, torch.int64):
            W[k] = t
        else:
            W[k] = (t.to(round_to) if round_to is not None and t.dim() == 2 else t).to(dtype)
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.numel()
    pos = torch.arange(T)
    eps = cfg["norm"]["eps"]
    x = W["embed"][tokens] * cfg["embedding"]["scale"]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        name, m = f"l{i}", layer["mixer"]
        if layer["type"] != "latent_attention":
            raise ValueError(layer["type"])
        h = norm_of(x, W, name + ".norm1")
        if m.get("kv_from") is None:
            kept[i] = latent_kv(h, W, name, m, eps, pos)
            c, kr = kept[i]
        else:
            c, kr = kept[m["kv_from"]]
        x = x + norm_of(latent_attention(h, W, name, m, c, kr, pos), W, name + ".norm1b")
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm_of(x, W, name + ".norm2")
            y = dense_ff(h, W, name + ".mlp") if mlp["kind"] == "dense" else moe_ff(h, W, name + ".mlp", mlp, margins_out)
            x = x + norm_of(y, W, name + ".norm2b")
        if cfg.get("token_side"):
            x = token_side(x, tokens, W, name, i, cfg["token_side"]["dim"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_of(x, W, "final.norm") @ W["head"].T

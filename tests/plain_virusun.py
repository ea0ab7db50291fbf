"""A plain, slow implementation of the Virusun design: whole sequences, no cache, one function a
mechanism, float64 on the CPU by default. It shares no code with the package; the tests compare
the engine with it.

A model is (config dict, tensors dict name -> torch tensor). Notation: h [T, W] is a sublayer's
input, rows are positions 0..T-1 of one sequence.
"""
from __future__ import annotations

import math

import torch


# The dtype an engine rounds to where it stores a result between kernels (keys and values in the
# cache, queries, the heads' results in front of an output projection, a feed-forward's hidden
# values and result); None: nothing is rounded. Set by forward(round_inputs=...).
ROUND_TO = None


# When a list: every recurrent mixer appends a tensor [T] to it, the smallest ratio over its heads of
# |S^T q| to | |S|^T |q| | at each position: how much of the read-out is left after cancellation. The
# norm that follows keeps the direction of the read-out and drops its size, so where the ratio is
# small the direction (behind a single token: the sign of k . q) is decided by rounding.
CANCELLATION = None


def _left_of_readout(S, q, o):
    return (o.norm() / ((S.abs().T @ q.abs()).norm() + 1e-30)).item()


def stored(x):
    return x if ROUND_TO is None else x.to(ROUND_TO).to(x.dtype)


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def lin(h, w, b=None):
    y = h @ w.T
    return y if b is None else y + b


def silu(z):
    return z * torch.sigmoid(z)


def causal_softmax(scores):
    """scores [..., T, T]: row i sees columns j <= i."""
    T = scores.shape[-1]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    return torch.softmax(scores.masked_fill(~mask, float("-inf")), dim=-1)


# ---- rotary angles with the ramp between scaled and unscaled frequencies ---------------------
def ramp_frequencies(dims, base, scaling):
    """(frequencies [dims/2], factor on sine and cosine)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, rot):
    """x [T, heads, D]; the first rot['dims'] entries of every head turn, entry i with i + dims/2."""
    dims = int(rot["dims"])
    if dims == 0:
        return x
    f, mag = ramp_frequencies(dims, float(rot["base"]), rot.get("scaling"))
    a = positions.to(torch.float64)[:, None] * f[None, :]
    cos, sin = (a.cos() * mag).to(x.dtype)[:, None, :], (a.sin() * mag).to(x.dtype)[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ---- mixers ----------------------------------------------------------------------------------
def diff_keys_values(h, m, t, pre, eps):
    """Keys after their norm [T, G, 2, dim] and values [T, G, vdim] of a differential layer."""
    T = h.shape[0]
    G, D, Dv = m["kv_heads"], m["dim"], m["vdim"]
    k = lin(h, t[pre + "k"], t[pre + "k.b"]).view(T, G, 2, D)
    k = rms(k, eps) * t[pre + "k.norm"]
    v = lin(h, t[pre + "v"], t[pre + "v.b"]).view(T, G, Dv)
    return stored(k), stored(v)


def differential_attention(h, m, t, pre, eps, kv):
    """``kv``: (keys, values) of the layer that owns them (this one, or the one it reads)."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = lin(h, t[pre + "q"], t[pre + "q.b"]).view(T, H, 2, D)
    q = stored(rms(q, eps) * t[pre + "q.norm"])
    k, v = kv
    rep = H // G
    k = k.repeat_interleave(rep, dim=1)                     # [T, H, 2, D]
    v = v.repeat_interleave(rep, dim=1)                     # [T, H, Dv]
    scores = torch.einsum("ihmd,jhmd->hmij", q, k) * m["scale"]
    p = causal_softmax(scores)                              # [H, 2, T, T]
    a = torch.einsum("hmij,jhe->ihme", p, v)                # [T, H, 2, Dv]
    lam = (torch.exp((t[pre + "lq1"] * t[pre + "lk1"]).sum())
           - torch.exp((t[pre + "lq2"] * t[pre + "lk2"]).sum()) + m["diff"])
    o = a[:, :, 0] - lam * a[:, :, 1]
    o = rms(o, eps) * (1.0 - m["diff"])
    o = o.reshape(T, H * Dv) * torch.sigmoid(lin(h, t[pre + "g"]))
    return lin(stored(o), t[pre + "o"], t[pre + "o.b"])


def rotary_attention(h, m, t, pre, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rms(lin(h, t[pre + "q"], t[pre + "q.b"]), eps) * t[pre + "q.norm"]
    k = rms(lin(h, t[pre + "k"], t[pre + "k.b"]), eps) * t[pre + "k.norm"]
    q = stored(rotate_half(q.view(T, H, D), pos, m["rot"]))
    k = stored(rotate_half(k.view(T, G, D), pos, m["rot"])).repeat_interleave(H // G, dim=1)
    v = stored(lin(h, t[pre + "v"], t[pre + "v.b"])).view(T, G, Dv).repeat_interleave(H // G, dim=1)
    p = causal_softmax(torch.einsum("ihd,jhd->hij", q, k) * m["scale"])
    o = torch.einsum("hij,jhe->ihe", p, v).reshape(T, H * Dv)
    return lin(stored(o), t[pre + "o"], t[pre + "o.b"])


def matrix_memory(h, m, t, pre, eps):
    """The matrix memory with exponential input gate and a running maximum that starts at 0."""
    T = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = lin(h, t[pre + "q"]).view(T, H, D) * D ** -0.5
    k = lin(h, t[pre + "k"]).view(T, H, D)
    v = lin(h, t[pre + "v"]).view(T, H, Dv)
    gi = cap * torch.tanh(lin(h, t[pre + "i"], t[pre + "i.b"]) / cap)                     # [T, H]
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh(lin(h, t[pre + "f"], t[pre + "f.b"]) / cap))
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    left = torch.ones(T)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=h.dtype)
        n = torch.zeros(D, dtype=h.dtype)
        mx = torch.zeros((), dtype=h.dtype)
        for s in range(T):
            m_new = torch.maximum(gf[s, hd] + mx, gi[s, hd])
            keep, take = torch.exp(gf[s, hd] + mx - m_new), torch.exp(gi[s, hd] - m_new)
            S = keep * S + take * torch.outer(k[s, hd], v[s, hd])
            n = keep * n + take * k[s, hd]
            mx = m_new
            den = torch.maximum((n @ q[s, hd]).abs(), torch.exp(-mx)) + 1e-6
            out[s, hd] = (S.T @ q[s, hd]) / den
            left[s] = min(left[s], _left_of_readout(S, q[s, hd], S.T @ q[s, hd]))
    if CANCELLATION is not None:
        CANCELLATION.append(left)
    o = rms(out, eps).reshape(T, H * Dv) * t[pre + "norm"] * torch.sigmoid(lin(h, t[pre + "g"]))
    return lin(stored(o), t[pre + "o"])


def short_conv(x, w):
    """x [T, C], w [C, taps]: y[s, c] = sum_j w[c, j] x[s - (taps - 1) + j, c], zeros before 0."""
    T, C = x.shape
    taps = w.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    return sum(xp[j:j + T] * w[:, j] for j in range(taps))


def gated_delta(h, m, t, pre, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(lin(h, t[pre + "q"]), t[pre + "q.conv"])).view(T, G, D)
    k = silu(short_conv(lin(h, t[pre + "k"]), t[pre + "k.conv"])).view(T, G, D)
    v = silu(short_conv(lin(h, t[pre + "v"]), t[pre + "v.conv"])).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(lin(h, t[pre + "b"]))                                                # [T, H]
    decay = torch.exp(-torch.exp(t[pre + "A_log"]) * torch.nn.functional.softplus(
        lin(h, t[pre + "a"]) + t[pre + "dt_bias"]))
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    left = torch.ones(T)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for s in range(T):
            S = decay[s, hd] * S
            u = beta[s, hd] * (v[s, hd] - S.T @ k[s, g])
            S = S + torch.outer(k[s, g], u)
            out[s, hd] = S.T @ q[s, g]
            left[s] = min(left[s], _left_of_readout(S, q[s, g], out[s, hd]))
    if CANCELLATION is not None:
        CANCELLATION.append(left)
    o = rms(out, eps) * t[pre + "norm"]
    o = o.reshape(T, H * Dv) * silu(lin(h, t[pre + "g"]))
    return lin(stored(o), t[pre + "o"])


def dense_ff(h, t, pre):
    return stored(lin(stored(silu(lin(h, t[pre + "gate"])) * lin(h, t[pre + "up"])), t[pre + "down"]))


# ---- the model ---------------------------------------------------------------------------------
def forward(config, tensors, tokens, dtype=torch.float64, return_layers=False, round_inputs=None,
            cancellation_out=None):
    """Logits [T, vocab] of one whole sequence (and the stream after every layer).
    ``round_inputs``: a dtype that every sublayer's input, and what an engine stores between
    kernels (see ROUND_TO), is rounded to, as an engine of that dtype rounds it (the stream itself
    is not rounded). ``cancellation_out``: a list that receives one tensor [T] a recurrent mixer (see
    CANCELLATION)."""
    global ROUND_TO, CANCELLATION
    ROUND_TO, CANCELLATION = round_inputs, cancellation_out
    try:
        return _forward(config, tensors, tokens, dtype, return_layers)
    finally:
        ROUND_TO = CANCELLATION = None


def _forward(config, tensors, tokens, dtype, return_layers):
    seen = stored

    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = float(config["norm"]["eps"])
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    kept, after = {}, []
    for i, layer in enumerate(config["layers"]):
        m, pre = layer["mixer"], f"l{i}.mix."
        kind = layer["type"]
        if kind == "attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = diff_keys_values(seen(x), m, t, pre, eps)
            y = differential_attention(seen(x), m, t, pre, eps, kept[i if src is None else src])
        elif kind == "parallel":
            y = (m["left_scale"] * rotary_attention(seen(x), m["left"], t, pre + "left.", eps)
                 + m["right_scale"] * matrix_memory(seen(x), m["right"], t, pre + "right.", eps))
        elif kind == "delta":
            y = gated_delta(seen(x), m, t, pre, eps)
        else:
            raise ValueError(kind)
        x = x + rms(y, eps) * t[f"l{i}.norm1"]
        if layer.get("mlp") is not None:
            x = x + rms(dense_ff(seen(x), t, f"l{i}.mlp."), eps) * t[f"l{i}.norm2"]
        after.append(x)
    logits = lin(seen(rms(x, eps) * t["final.norm"]), t["head"])
    return (logits, torch.stack(after)) if return_layers else logits

"""The kernels of the Virusun mixers, each alone, against the plain functions of
tests/plain_virusun.py or a few lines of float64 arithmetic: odd sizes, positions beyond a
thousand, pages in shuffled order, sequences cut at every kind of place, state slots in any order."""
import math

import pytest
import torch

import plain_virusun as pv

pytestmark = pytest.mark.gpu


def dev(t, dtype=torch.float32):
    return t.to("cuda", dtype).contiguous()


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode,rot,scaling,own", [("head", 0, None, True), ("whole", 12, (4.0, 64, 8.0, 1.0), True),
                                                 ("whole", 20, None, True), (None, 8, (2.0, 32, 4.0, 0.5), True),
                                                 ("head", 0, None, False)])
def test_prepare_queries_keys_values(gpu_device, dtype, mode, rot, scaling, own):
    from pytriton_llama_amd import ops
    from pytriton_llama_amd.parts.rotary import ramp_inv_freq
    torch.manual_seed(3)
    T, Hq, Hk, Hv, Dk, Dv, P, pages = 37, 6, 4, 2, 20, 12, 4, 40
    nq, nk, nv = Hq * Dk, Hk * Dk, Hv * Dv
    pad = 5
    p = torch.randn(T, pad + nq + nk + nv + 3, dtype=torch.float64)
    qb, kb, vb = torch.randn(nq, dtype=torch.float64), torch.randn(nk, dtype=torch.float64), torch.randn(nv, dtype=torch.float64)
    whole = mode == "whole"
    qw = 1 + 0.3 * torch.randn(nq if whole else Dk, dtype=torch.float64)
    kw = 1 + 0.3 * torch.randn(nk if whole else Dk, dtype=torch.float64)
    positions = torch.randint(0, 3000, (T,))
    eps = 1e-5
    # plain
    q = p[:, pad:pad + nq] + qb
    k = p[:, pad + nq:pad + nq + nk] + kb
    v = p[:, pad + nq + nk:pad + nq + nk + nv] + vb
    if mode == "whole":
        q, k = pv.rms(q, eps) * qw, pv.rms(k, eps) * kw
    q, k = q.view(T, Hq, Dk), k.view(T, Hk, Dk)
    if mode == "head":
        q, k = pv.rms(q, eps) * qw, pv.rms(k, eps) * kw
    rot_cfg = {"dims": rot, "base": 500.0}
    if scaling:
        rot_cfg["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    q, k = pv.rotate_half(q, positions, rot_cfg), pv.rotate_half(k, positions, rot_cfg)
    # kernel
    inv_freq, mag = None, 1.0
    if rot:
        if scaling:
            inv_freq, mag = ramp_inv_freq(500.0, rot, *scaling)
        else:
            inv_freq = (500.0 ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)).float()
        inv_freq = inv_freq.cuda()
    slots = torch.randperm(pages * P)[:T].to(torch.int32)
    k_cache = torch.zeros(pages, Hk, P, Dk, dtype=dtype, device="cuda")
    v_cache = torch.zeros(pages, Hv, P, Dv, dtype=dtype, device="cuda")
    q_out = torch.empty(T, Hq, Dk, dtype=dtype, device="cuda")
    code = {None: ops.NORM_NONE, "head": ops.NORM_HEAD, "whole": ops.NORM_WHOLE}[mode]
    ops.qkv_prepare(q_out, dev(p), pad, pad + nq if own else -1, pad + nq + nk, dev(qb), dev(kb), dev(vb), code,
                    dev(qw) if mode else None, dev(kw) if mode else None, eps, rot, inv_freq, mag,
                    positions.to(torch.int32).cuda(), slots.cuda(), k_cache, v_cache, Hq, Hk, Hv, Dk, Dv, P)
    # angles are float32: at position 3000 half an ulp of the angle is 1.2e-4
    tol = (2e-4 if rot else 2e-5) if dtype == torch.float32 else 2e-2
    assert float((q_out.double().cpu() - q).abs().max()) < tol * float(q.abs().max())
    if not own:
        assert float(k_cache.abs().max()) == 0 and float(v_cache.abs().max()) == 0
        return
    page, at = slots.long() // P, slots.long() % P
    got_k = k_cache.double().cpu()[page, :, at]            # [T, Hk, Dk]
    got_v = v_cache.double().cpu()[page, :, at]
    assert float((got_k - k).abs().max()) < tol * float(k.abs().max())
    assert float((got_v - v.view(T, Hv, Dv)).abs().max()) < tol * float(v.abs().max())


def paged(x, page_size, pages, order):
    """x [n, heads, size] of one sequence -> a pool [pages, heads, page_size, size] with the
    sequence's pages at ``order``."""
    n, H, D = x.shape
    pool = torch.randn(pages, H, page_size, D, dtype=x.dtype) * 5      # what lies in pages of others
    for i in range(n):
        pool[order[i // page_size], :, i % page_size] = x[i]
    return pool


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("maps,H,G,Dk,Dv", [(1, 6, 3, 24, 40), (2, 4, 2, 20, 12), (2, 3, 3, 16, 16), (1, 2, 1, 136, 8)])
def test_attention_with_keys_and_values_of_different_sizes(gpu_device, dtype, maps, H, G, Dk, Dv):
    """Two sequences in one batch (a portion behind a cached prefix, and a single decoded token
    behind 300 keys), pages in shuffled order; one far key (position 3, and the last of a page) is
    made to stand out for some queries, so that losing it would show."""
    from pytriton_llama_amd import ops
    from pytriton_llama_amd.engine.batch import work_items
    torch.manual_seed(5)
    P, pages = 8, 80
    lens, qlens = [130, 301], [50, 1]
    scale = 0.3
    qs, ks, vs, outs = [], [], [], []
    for n, ql in zip(lens, qlens):
        k = torch.randn(n, G * maps, Dk, dtype=torch.float64)
        v = torch.randn(n, G, Dv, dtype=torch.float64)
        q = torch.randn(ql, H * maps, Dk, dtype=torch.float64)
        for far in (3, P * 5 - 1, P * 5):
            k[far] *= 3.0
            q[-1, 0] = k[far, 0] * 2.0             # the last query's first head looks at the far key
        if dtype == torch.bfloat16:
            q, k, v = (t.bfloat16().double() for t in (q, k, v))
        out = torch.zeros(ql, H * maps, Dv, dtype=torch.float64)
        for j in range(H * maps):
            vh = (j // maps) // (H // G)
            kh = vh * maps + j % maps
            s = (q[:, j] @ k[:, kh].T) * scale                                  # [ql, n]
            pos = torch.arange(n - ql, n)[:, None]
            s = s.masked_fill(torch.arange(n)[None, :] > pos, float("-inf"))
            out[:, j] = torch.softmax(s, -1) @ v[:, vh]
        qs.append(q), ks.append(k), vs.append(v), outs.append(out)
    order = torch.randperm(pages).tolist()
    need = [-(-n // P) for n in lens]
    tables = [order[:need[0]], order[need[0]:need[0] + need[1]]]
    k_pool = torch.randn(pages, G * maps, P, Dk, dtype=torch.float64) * 5
    v_pool = torch.randn(pages, G, P, Dv, dtype=torch.float64) * 5
    for k, v, table in zip(ks, vs, tables):
        for i in range(k.shape[0]):
            k_pool[table[i // P], :, i % P] = k[i]
            v_pool[table[i // P], :, i % P] = v[i]
    width = max(need)
    bt = torch.full((2, width), -1, dtype=torch.int32)
    for r, table in enumerate(tables):
        bt[r, :len(table)] = torch.tensor(table, dtype=torch.int32)
    q_all = torch.cat(qs)
    ws, wo = work_items(qlens, lens, 0, 16)
    for out_dtype in ([torch.float32] if dtype == torch.float32 else [torch.float32, torch.bfloat16]):
        out = torch.empty(q_all.shape[0], H * maps, Dv, dtype=out_dtype, device="cuda")
        ops.attention_generic_kv(out, dev(q_all, dtype), dev(k_pool, dtype), dev(v_pool, dtype), i32([0, 50, 51]),
                                 i32(lens), bt.cuda(), torch.from_numpy(ws).cuda(), torch.from_numpy(wo).cuda(),
                                 scale, maps)
        want = torch.cat(outs)
        tol = 2e-5 if out_dtype == torch.float32 else 1e-2
        assert float((out.double().cpu() - want).abs().max()) < tol * float(want.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("maps,per_head,act", [(2, None, "sigmoid"), (1, True, "sigmoid"), (1, False, "silu"), (2, None, None)])
def test_heads_normed_and_gated(gpu_device, dtype, maps, per_head, act):
    from pytriton_llama_amd import ops
    torch.manual_seed(7)
    T, H, Dv, lam, mult, eps = 29, 5, 72, 0.37, 0.55, 1e-5
    a = torch.randn(T, H * maps, Dv, dtype=torch.float64)
    gate = torch.randn(T, 11 + H * Dv, dtype=torch.float64)
    w = None if per_head is None else 1 + 0.2 * torch.randn(H * Dv if per_head else Dv, dtype=torch.float64)
    o = a.view(T, H, maps, Dv)
    o = o[:, :, 0] - lam * o[:, :, 1] if maps == 2 else o[:, :, 0]
    o = pv.rms(o, eps) * mult
    if w is not None:
        o = o * (w.view(H, Dv) if per_head else w)
    g = gate[:, 11:].view(T, H, Dv)
    if act == "sigmoid":
        o = o * torch.sigmoid(g)
    elif act == "silu":
        o = o * pv.silu(g)
    out = torch.empty(T, H * Dv, dtype=dtype, device="cuda")
    code = {None: ops.GATE_NONE, "sigmoid": ops.GATE_SIGMOID, "silu": ops.GATE_SILU}[act]
    ops.head_norm_gate(out, dev(a), maps, lam, dev(w) if w is not None else None, bool(per_head), mult,
                       dev(gate) if act else None, 11, code, eps)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert float((out.double().cpu().view(T, H, Dv) - o).abs().max()) < tol * float(o.abs().max())


def cut(total, sizes):
    out, lo, i = [], 0, 0
    while lo < total:
        hi = min(total, lo + sizes[i % len(sizes)])
        out.append((lo, hi))
        lo, i = hi, i + 1
    return out


@pytest.mark.parametrize("G,H,D,Dv,taps", [(1, 2, 16, 16, 4), (3, 3, 20, 36, 3), (2, 6, 40, 12, 2), (2, 2, 8, 50, 1),
                                           (1, 1, 200, 24, 2), (1, 2, 136, 8, 3)])
def test_delta_rule_in_portions_and_batches(gpu_device, G, H, D, Dv, taps):
    """Three sequences of unequal length that advance together in portions of changing size (down
    to one token, shorter than the convolution), in state slots used in any order; a slot is then
    cleared and used by another sequence."""
    from pytriton_llama_amd import ops
    torch.manual_seed(11)
    C = 2 * G * D + H * Dv
    cols = C + 2 * H
    lens = [61, 23, 40]
    eps = 1e-5
    cw = torch.randn(C, taps, dtype=torch.float64) * 0.5
    A_log, dt_bias = torch.rand(H, dtype=torch.float64) * 2 - 2, torch.randn(H, dtype=torch.float64)
    ps = [torch.randn(n, cols, dtype=torch.float64) for n in lens]

    def plain(p):
        T = p.shape[0]
        x = pv.silu(pv.short_conv(p[:, :C], cw))
        q, k, v = x[:, :G * D].view(T, G, D), x[:, G * D:2 * G * D].view(T, G, D), x[:, 2 * G * D:].view(T, H, Dv)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(p[:, C + H:])
        decay = torch.exp(-torch.exp(A_log) * torch.nn.functional.softplus(p[:, C:C + H] + dt_bias))
        out = torch.zeros(T, H, Dv, dtype=torch.float64)
        for h in range(H):
            S = torch.zeros(D, Dv, dtype=torch.float64)
            for s in range(T):
                S = decay[s, h] * S
                S = S + torch.outer(k[s, h // (H // G)], beta[s, h] * (v[s, h] - S.T @ k[s, h // (H // G)]))
                out[s, h] = S.T @ q[s, h // (H // G)]
        return out

    want = [plain(p) for p in ps]
    tail_off = ops.recurrent_state_floats(H, D, Dv)
    state = torch.randn(6, tail_off + (taps - 1) * C, device="cuda")         # slots hold old values
    slot_of = [4, 0, 2]
    for s in slot_of:
        state[s].zero_()
    cuts = [cut(lens[0], (7, 1, 1, 2, 19)), cut(lens[1], (1, 2, 1, 30)), cut(lens[2], (16, 3, 1))]
    got = [torch.zeros_like(w) for w in want]
    cw_d, A_d, dt_d = dev(cw), dev(A_log), dev(dt_bias)

    def step(parts):
        """parts: [(sequence, lo, hi)] of one batch."""
        p = torch.cat([ps[i][lo:hi] for i, lo, hi in parts])
        starts = [0]
        for _, lo, hi in parts:
            starts.append(starts[-1] + hi - lo)
        q_start, slots = i32(starts), i32([slot_of[i] for i, _, _ in parts])
        pd = dev(p)
        q, k, v = ops.conv_prepare(pd, 0, cw_d, state, tail_off, q_start, slots, G, H, D, Dv, D ** -0.5)
        ops.conv_tail_update(pd, 0, C, taps, state, tail_off, q_start, slots)
        o = ops.delta_scan(q, k, v, pd, C, C + H, A_d, dt_d, state, q_start, slots).double().cpu()
        for j, (i, lo, hi) in enumerate(parts):
            got[i][lo:hi] = o[starts[j]:starts[j + 1]]

    for r in range(max(len(c) for c in cuts)):
        parts = [(i, *cuts[i][r]) for i in (2, 0, 1) if r < len(cuts[i])]
        step(parts)
    for g, w in zip(got, want):
        assert float((g - w).abs().max()) < 2e-5 * float(w.abs().max())
    # a slot that another sequence has filled, cleared as the engine clears it at admission
    state[slot_of[0]].zero_()
    slot_of[1] = slot_of[0]
    got[1].zero_()
    step([(1, 0, lens[1])])
    assert float((got[1] - want[1]).abs().max()) < 2e-5 * float(want[1].abs().max())


@pytest.mark.parametrize("H,D,Dv,cap", [(2, 16, 16, 12.0), (3, 20, 36, 4.0), (1, 48, 40, 30.0), (5, 8, 8, 1.5),
                                        (1, 256, 20, 8.0), (1, 176, 8, 6.0)])
def test_matrix_memory_in_portions_and_batches(gpu_device, H, D, Dv, cap):
    from pytriton_llama_amd import ops
    torch.manual_seed(13)
    lens = [57, 18, 33]
    q_off, k_off, v_off, i_off, f_off = 3, 3 + H * D, 3 + 2 * H * D, 3 + 2 * H * D + H * Dv, 3 + 2 * H * D + H * Dv + H
    cols = f_off + H + 2
    ib, fb = torch.randn(H, dtype=torch.float64), torch.randn(H, dtype=torch.float64) + 2
    ps = []
    for n in lens:
        p = torch.randn(n, cols, dtype=torch.float64)
        p[:, i_off:f_off + H] *= 4.0           # gates that reach their cap, forget gates near 0 and near 1
        ps.append(p)

    def plain(p):
        T = p.shape[0]
        q = p[:, q_off:k_off].view(T, H, D) * D ** -0.5
        k, v = p[:, k_off:v_off].view(T, H, D), p[:, v_off:i_off].view(T, H, Dv)
        gi = cap * torch.tanh((p[:, i_off:f_off] + ib) / cap)
        gf = torch.nn.functional.logsigmoid(cap * torch.tanh((p[:, f_off:f_off + H] + fb) / cap))
        out = torch.zeros(T, H, Dv, dtype=torch.float64)
        for h in range(H):
            S, n, m = torch.zeros(D, Dv, dtype=torch.float64), torch.zeros(D, dtype=torch.float64), torch.zeros((), dtype=torch.float64)
            for s in range(T):
                m_new = torch.maximum(gf[s, h] + m, gi[s, h])
                keep, take = torch.exp(gf[s, h] + m - m_new), torch.exp(gi[s, h] - m_new)
                S, n, m = keep * S + take * torch.outer(k[s, h], v[s, h]), keep * n + take * k[s, h], m_new
                out[s, h] = S.T @ q[s, h] / (torch.maximum((n @ q[s, h]).abs(), torch.exp(-m)) + 1e-6)
        return out

    want = [plain(p) for p in ps]
    state = torch.randn(5, ops.recurrent_state_floats(H, D, Dv) + 7, device="cuda")
    slot_of = [3, 1, 0]
    for s in slot_of:
        state[s].zero_()
    cuts = [cut(lens[0], (5, 1, 1, 17, 2)), cut(lens[1], (1, 1, 16)), cut(lens[2], (16, 1, 3))]
    got = [torch.zeros_like(w) for w in want]
    ib_d, fb_d = dev(ib), dev(fb)
    for r in range(max(len(c) for c in cuts)):
        parts = [(i, *cuts[i][r]) for i in (1, 2, 0) if r < len(cuts[i])]
        p = dev(torch.cat([ps[i][lo:hi] for i, lo, hi in parts]))
        starts = [0]
        for _, lo, hi in parts:
            starts.append(starts[-1] + hi - lo)
        o = ops.memory_scan(p, q_off, k_off, v_off, i_off, f_off, ib_d, fb_d, cap, D ** -0.5, state, i32(starts),
                            i32([slot_of[i] for i, _, _ in parts]), H, D, Dv).double().cpu()
        for j, (i, lo, hi) in enumerate(parts):
            got[i][lo:hi] = o[starts[j]:starts[j + 1]]
    for g, w in zip(got, want):
        assert float((g - w).abs().max()) < 3e-5 * float(w.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_of_a_weighted_sum_into_the_stream(gpu_device, dtype):
    from pytriton_llama_amd import ops
    torch.manual_seed(17)
    T, W, eps = 21, 200, 1e-5
    stream = torch.randn(T, W, dtype=torch.float64)
    y1, y2 = torch.randn(T, W, dtype=torch.float64), torch.randn(T, W, dtype=torch.float64)
    bias, w = torch.randn(W, dtype=torch.float64), 1 + 0.2 * torch.randn(W, dtype=torch.float64)
    for second, with_bias in ((True, True), (False, True), (True, False), (False, False)):
        y = 1.2 * y1 + (0.7 * y2 if second else 0) + (1.2 * bias if with_bias else 0)
        want = stream + pv.rms(y, eps) * w
        s = dev(stream)
        copy = ops.stream_add_rmsnorm_sum(s, dev(y1), 1.2, dev(y2) if second else None, 0.7,
                                          dev(bias) if with_bias else None, 1.2, dev(w), eps, dtype, True)
        assert float((s.double().cpu() - want).abs().max()) < 1e-5
        assert copy.dtype == dtype
        assert float((copy.double().cpu() - want).abs().max()) < (1e-5 if dtype == torch.float32 else 3e-2)
    out = ops.stream_rmsnorm(dev(stream), dev(w), eps, dtype)
    assert float((out.double().cpu() - pv.rms(stream, eps) * w).abs().max()) < (1e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("maps,H,G,Dk,Dv", [(1, 6, 3, 32, 48), (2, 4, 2, 48, 96), (2, 10, 2, 16, 16), (1, 2, 1, 144, 32)])
@pytest.mark.parametrize("splits", [1, 3, 8])
def test_decoding_attention_with_keys_split_over_workgroups(gpu_device, dtype, maps, H, G, Dk, Dv, splits):
    """Single query tokens of three sequences (1, 130 and 333 keys; pages in shuffled order), the
    keys of each cut into ``splits`` parts; for one head the key at a page's last place is made to
    stand out."""
    from pytriton_llama_amd import ops
    torch.manual_seed(19)
    P, pages, scale = 8, 80, 0.25
    lens = [1, 130, 333]
    order = torch.randperm(pages).tolist()
    k_pool = torch.randn(pages, G * maps, P, Dk, dtype=torch.float64) * 5
    v_pool = torch.randn(pages, G, P, Dv, dtype=torch.float64) * 5
    bt = torch.full((3, -(-max(lens) // P)), -1, dtype=torch.int32)
    qs, want, at = [], [], 0
    for r, n in enumerate(lens):
        k = torch.randn(n, G * maps, Dk, dtype=torch.float64)
        v = torch.randn(n, G, Dv, dtype=torch.float64)
        q = torch.randn(1, H * maps, Dk, dtype=torch.float64)
        if n > P:
            k[P * 2 - 1] *= 3.0
            q[0, 0] = k[P * 2 - 1, 0] * 2.0
        if dtype == torch.bfloat16:
            q, k, v = (t.bfloat16().double() for t in (q, k, v))
        out = torch.zeros(1, H * maps, Dv, dtype=torch.float64)
        for j in range(H * maps):
            vh = (j // maps) // (H // G)
            out[0, j] = torch.softmax((q[0, j] @ k[:, vh * maps + j % maps].T) * scale, -1) @ v[:, vh]
        table = order[at:at + -(-n // P)]
        at += len(table)
        bt[r, :len(table)] = torch.tensor(table, dtype=torch.int32)
        for i in range(n):
            k_pool[table[i // P], :, i % P] = k[i]
            v_pool[table[i // P], :, i % P] = v[i]
        qs.append(q), want.append(out)
    want = torch.cat(want)
    for out_dtype in ([torch.float32] if dtype == torch.float32 else [torch.float32, torch.bfloat16]):
        out = torch.empty(3, H * maps, Dv, dtype=out_dtype, device="cuda")
        ops.attention_decode_kv(out, dev(torch.cat(qs), dtype), dev(k_pool, dtype), dev(v_pool, dtype),
                                i32([0, 1, 2, 3]), i32(lens), bt.cuda(), 3, scale, maps, splits)
        tol = 2e-5 if out_dtype == torch.float32 else 1e-2
        assert float((out.double().cpu() - want).abs().max()) < tol * float(want.abs().max())


@pytest.mark.parametrize("maps,H,G,Dk,Dv", [(1, 4, 2, 64, 32), (2, 4, 2, 32, 64), (2, 2, 2, 64, 128), (1, 3, 1, 128, 96),
                                            (2, 8, 4, 96, 32)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_matrix_core_attention_for_prompt_portions(gpu_device, maps, H, G, Dk, Dv, out_dtype):
    """Three sequences (a whole prompt of 200 tokens, 70 tokens behind a cached prefix of 450 that
    starts inside a page, 3 tokens behind 64), pages in shuffled order; the key at a page's last
    place stands out for a few queries. One workgroup a block, and few that share the list."""
    from pytriton_llama_amd import ops
    from pytriton_llama_amd.engine.batch import work_items
    torch.manual_seed(23)
    P, pages, scale = 16, 64, 0.2
    lens, qlens = [200, 520, 67], [200, 70, 3]
    order = torch.randperm(pages).tolist()
    k_pool = (torch.randn(pages, G * maps, P, Dk, dtype=torch.float64) * 5).bfloat16().double()
    v_pool = (torch.randn(pages, G, P, Dv, dtype=torch.float64) * 5).bfloat16().double()
    bt = torch.full((3, -(-max(lens) // P)), -1, dtype=torch.int32)
    qs, want, at = [], [], 0
    for r, (n, ql) in enumerate(zip(lens, qlens)):
        k = torch.randn(n, G * maps, Dk, dtype=torch.float64)
        v = torch.randn(n, G, Dv, dtype=torch.float64)
        q = torch.randn(ql, H * maps, Dk, dtype=torch.float64)
        k[P * 2 - 1] *= 2.0
        q[-1, 0] = k[P * 2 - 1, 0] * 1.5
        q, k, v = (t.bfloat16().double() for t in (q, k, v))
        out = torch.zeros(ql, H * maps, Dv, dtype=torch.float64)
        for j in range(H * maps):
            vh = (j // maps) // (H // G)
            s = (q[:, j] @ k[:, vh * maps + j % maps].T) * scale
            s = s.masked_fill(torch.arange(n)[None, :] > torch.arange(n - ql, n)[:, None], float("-inf"))
            out[:, j] = torch.softmax(s, -1) @ v[:, vh]
        table = order[at:at + -(-n // P)]
        at += len(table)
        bt[r, :len(table)] = torch.tensor(table, dtype=torch.int32)
        for i in range(n):
            k_pool[table[i // P], :, i % P] = k[i]
            v_pool[table[i // P], :, i % P] = v[i]
        qs.append(q), want.append(out)
    want = torch.cat(want)
    ws, wo = work_items(qlens, lens, 0, 64)
    for groups in (len(ws), 2):
        out = torch.empty(sum(qlens), H * maps, Dv, dtype=out_dtype, device="cuda")
        ops.attention_prefill_mfma_kv(out, dev(torch.cat(qs), torch.bfloat16), dev(k_pool, torch.bfloat16),
                                      dev(v_pool, torch.bfloat16), i32([0, 200, 270, 273]), i32(lens), bt.cuda(),
                                      torch.from_numpy(ws).cuda(), torch.from_numpy(wo).cuda(), scale, maps, groups)
        # probabilities are rounded to bfloat16 for the second product
        assert float((out.double().cpu() - want).abs().max()) < 1.5e-2 * float(want.abs().max())


@pytest.mark.parametrize("H,D,Dv,cap", [(2, 32, 24, 10.0), (1, 72, 40, 3.0)])
def test_matrix_memory_of_long_portions_in_segments(gpu_device, H, D, Dv, cap):
    """Portions long enough to be worked on in segments side by side (with a last segment that is not
    full, and a short sequence and a single token in the same step), then more tokens one by one
    from the state the segments left; against the walk in one chain."""
    from pytriton_llama_amd import ops
    torch.manual_seed(29)
    lens = [700, 30, 1, 530]
    q_off, k_off, v_off, i_off, f_off = 0, H * D, 2 * H * D, 2 * H * D + H * Dv, 2 * H * D + H * Dv + H
    cols = f_off + H
    ib, fb = torch.randn(H, dtype=torch.float64), torch.randn(H, dtype=torch.float64) + 2
    ps = []
    for n in lens:
        p = torch.randn(n + 5, cols, dtype=torch.float64)
        p[:, i_off:] *= 3.0
        ps.append(p)

    def plain(p):
        T = p.shape[0]
        q = p[:, q_off:k_off].view(T, H, D) * D ** -0.5
        k, v = p[:, k_off:v_off].view(T, H, D), p[:, v_off:i_off].view(T, H, Dv)
        gi = cap * torch.tanh((p[:, i_off:f_off] + ib) / cap)
        gf = torch.nn.functional.logsigmoid(cap * torch.tanh((p[:, f_off:f_off + H] + fb) / cap))
        out = torch.zeros(T, H, Dv, dtype=torch.float64)
        for h in range(H):
            S, n, m = torch.zeros(D, Dv, dtype=torch.float64), torch.zeros(D, dtype=torch.float64), torch.zeros((), dtype=torch.float64)
            for s in range(T):
                m_new = torch.maximum(gf[s, h] + m, gi[s, h])
                keep, take = torch.exp(gf[s, h] + m - m_new), torch.exp(gi[s, h] - m_new)
                S, n, m = keep * S + take * torch.outer(k[s, h], v[s, h]), keep * n + take * k[s, h], m_new
                out[s, h] = S.T @ q[s, h] / (torch.maximum((n @ q[s, h]).abs(), torch.exp(-m)) + 1e-6)
        return out

    want = [plain(p) for p in ps]
    state = torch.randn(6, ops.recurrent_state_floats(H, D, Dv), device="cuda")
    slot_of = [2, 5, 0, 3]
    for s in slot_of:
        state[s].zero_()
    ib_d, fb_d = dev(ib), dev(fb)

    def run(parts, longest):
        p = dev(torch.cat([ps[i][lo:hi] for i, lo, hi in parts]))
        starts = [0]
        for _, lo, hi in parts:
            starts.append(starts[-1] + hi - lo)
        o = ops.memory_scan(p, q_off, k_off, v_off, i_off, f_off, ib_d, fb_d, cap, D ** -0.5, state, i32(starts),
                            i32([slot_of[i] for i, _, _ in parts]), H, D, Dv, longest).double().cpu()
        return [o[starts[j]:starts[j + 1]] for j in range(len(parts))]

    assert max(lens) >= ops.MEMORY_SEGMENTS_FROM
    got = run([(2, 0, 1), (0, 0, 700), (1, 0, 30), (3, 0, 530)], 700)
    for g, i in zip(got, (2, 0, 1, 3)):
        assert float((g - want[i][:lens[i]]).abs().max()) < 3e-5 * float(want[i].abs().max())
    # five more tokens of each, one by one (the walk in one chain), from the states the segments left
    for t in range(5):
        got = run([(i, lens[i] + t, lens[i] + t + 1) for i in range(4)], 1)
        for i, g in enumerate(got):
            assert float((g[0] - want[i][lens[i] + t]).abs().max()) < 3e-5 * float(want[i].abs().max())


@pytest.mark.parametrize("G,H,D,Dv,taps", [(1, 2, 32, 24, 3), (2, 2, 40, 72, 2)])
def test_delta_rule_of_long_portions_in_segments(gpu_device, G, H, D, Dv, taps):
    """Portions long enough to be worked on in segments side by side (a last segment that is not
    full; a short sequence and a single token in the same step), then more tokens one by one from
    the state the segments left; against the walk in one chain."""
    from pytriton_llama_amd import ops
    torch.manual_seed(31)
    C = 2 * G * D + H * Dv
    cols = C + 2 * H
    lens = [900, 20, 1, 300]
    cw = torch.randn(C, taps, dtype=torch.float64) * 0.5
    A_log, dt_bias = torch.rand(H, dtype=torch.float64) * 2 - 3, torch.randn(H, dtype=torch.float64)
    ps = [torch.randn(n + 4, cols, dtype=torch.float64) for n in lens]

    def plain(p):
        T = p.shape[0]
        x = pv.silu(pv.short_conv(p[:, :C], cw))
        q, k, v = x[:, :G * D].view(T, G, D), x[:, G * D:2 * G * D].view(T, G, D), x[:, 2 * G * D:].view(T, H, Dv)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(p[:, C + H:])
        decay = torch.exp(-torch.exp(A_log) * torch.nn.functional.softplus(p[:, C:C + H] + dt_bias))
        out = torch.zeros(T, H, Dv, dtype=torch.float64)
        for h in range(H):
            S = torch.zeros(D, Dv, dtype=torch.float64)
            for s in range(T):
                S = decay[s, h] * S
                S = S + torch.outer(k[s, h // (H // G)], beta[s, h] * (v[s, h] - S.T @ k[s, h // (H // G)]))
                out[s, h] = S.T @ q[s, h // (H // G)]
        return out

    want = [plain(p) for p in ps]
    tail_off = ops.recurrent_state_floats(H, D, Dv)
    state = torch.randn(6, tail_off + (taps - 1) * C, device="cuda")
    slot_of = [1, 4, 0, 5]
    for s in slot_of:
        state[s].zero_()
    cw_d, A_d, dt_d = dev(cw), dev(A_log), dev(dt_bias)

    def run(parts, longest):
        p = dev(torch.cat([ps[i][lo:hi] for i, lo, hi in parts]))
        starts = [0]
        for _, lo, hi in parts:
            starts.append(starts[-1] + hi - lo)
        q_start, slots = i32(starts), i32([slot_of[i] for i, _, _ in parts])
        q, k, v = ops.conv_prepare(p, 0, cw_d, state, tail_off, q_start, slots, G, H, D, Dv, D ** -0.5)
        ops.conv_tail_update(p, 0, C, taps, state, tail_off, q_start, slots)
        o = ops.delta_scan(q, k, v, p, C, C + H, A_d, dt_d, state, q_start, slots, longest).double().cpu()
        return [o[starts[j]:starts[j + 1]] for j in range(len(parts))]

    assert max(lens) >= ops.DELTA_SEGMENTS_FROM
    got = run([(2, 0, 1), (0, 0, 900), (1, 0, 20), (3, 0, 300)], 900)
    for g, i in zip(got, (2, 0, 1, 3)):
        assert float((g - want[i][:lens[i]]).abs().max()) < 3e-5 * float(want[i].abs().max())
    for t in range(4):
        got = run([(i, lens[i] + t, lens[i] + t + 1) for i in range(4)], 1)
        for i, g in enumerate(got):
            assert float((g[0] - want[i][lens[i] + t]).abs().max()) < 3e-5 * float(want[i].abs().max())

"""Each new mechanism alone, kernel against a plain float32 computation of the same thing:
Dynamic-Tanh norms on the float32 stream, the RMS-norm sum, the gated token input, the latent
cache write with its rotation of neighbouring pairs, per-head products, routing and the routed
experts. Sizes are odd on purpose; bfloat16 runs compare with the rounded operands."""
import math

import pytest
import torch

import plain_rubasun as P

pytestmark = pytest.mark.gpu


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * std


def close(got, want, tol):
    return float((got.float().cpu() - want).abs().max() / want.abs().max()) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_stream_sum_between_two_dynamic_tanh_norms(gpu_device, dtype):
    from pytriton_llama_amd import ops
    T, H = 37, 72
    stream, y = rnd(T, H, seed=1, std=3.0), rnd(T, H, seed=2, std=2.0).to(dtype)
    w1, b1, w2, b2 = rnd(H, seed=3), rnd(H, seed=4, std=0.2), rnd(H, seed=5), rnd(H, seed=6, std=0.2)
    want_stream = stream + P.dyt(y.float(), w1, b1, 0.7)
    want_out = P.dyt(want_stream, w2, b2, 1.3)
    dev = lambda t: t.to(gpu_device)
    s = dev(stream.clone())
    out, copy = ops.stream_add_dyt(s, dev(y), (dev(w1), dev(b1), 0.7), (dev(w2), dev(b2), 1.3), dtype, True)
    assert s.dtype == torch.float32 and close(s, want_stream, 1e-6)
    assert out.dtype == dtype and close(out, want_out, 1e-6 if dtype == torch.float32 else 8e-3)
    assert close(copy, want_stream, 1e-6 if dtype == torch.float32 else 8e-3)
    # a plain sum, and the norm alone
    s2 = dev(stream.clone())
    ops.stream_add_dyt(s2, dev(y), None, None, dtype)
    assert close(s2, stream + y.float(), 1e-6)
    alone = ops.dyt(dev(stream), dev(w2), dev(b2), 1.3, dtype)
    assert close(alone, P.dyt(stream, w2, b2, 1.3), 1e-6 if dtype == torch.float32 else 8e-3)


def test_stream_sum_of_an_rms_normed_row_and_scaled_embedding(gpu_device):
    from pytriton_llama_amd import ops
    T, H, V = 9, 300, 50
    stream, y, w = rnd(T, H, seed=1), rnd(T, H, seed=2, std=5.0), rnd(H, seed=3)
    s = stream.clone().to(gpu_device)
    ops.stream_add_rmsnorm(s, y.to(gpu_device), w.to(gpu_device), 1e-3)
    assert close(s, stream + P.rms(y, 1e-3) * w, 2e-6)
    table = rnd(V, H, seed=4).to(torch.bfloat16)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    e = ops.embedding_scaled(table.to(gpu_device), ids.to(gpu_device), 2.5)
    assert e.dtype == torch.float32 and torch.equal(e.cpu(), table.float()[ids.long()] * 2.5)
    z, side = rnd(4, 6, seed=5), rnd(V, 18, seed=6)
    g = ops.gelu_gather_mul(z.to(gpu_device), side.to(gpu_device), ids.to(gpu_device), 6)
    assert close(g, P.gelu_tanh(z) * side[ids.long()][:, 6:12], 2e-6)


@pytest.mark.parametrize("dims", [12, 8, 0])
def test_latent_cache_write_and_rotation_of_pairs(gpu_device, dims):
    """Positions beyond a thousand, a rotated part that turns wholly, in part or not at all, a
    token without a slot (a padding row) that must leave the cache alone. The plain values are
    float64; a float32 angle at position 1,500 is good to 1e-4 radians, hence the bound."""
    from pytriton_llama_amd import ops
    from pytriton_llama_amd.parts.latent_attention import paired_inv_freq
    T, H, dn, dr, R, page = 6, 3, 10, 12, 20, 4
    D = R + dr
    proj = rnd(T, H * (dn + dr) + D + 5, seed=1)
    pos = torch.tensor([0, 1, 7, 1500, 33, 2], dtype=torch.int32)
    slots = torch.tensor([5, 0, 11, 2, -1, 9], dtype=torch.int32)
    cw = rnd(R, seed=2)
    inv = paired_inv_freq(777.0, dims) if dims else None
    q = torch.zeros(T, H, D, device=gpu_device)
    cache = torch.full((3, 1, page, D), 9.0, device=gpu_device)
    ops.latent_prepare(q, proj.to(gpu_device), 0, H * (dn + dr), pos.to(gpu_device),
                       inv.to(gpu_device) if dims else None, cw.to(gpu_device), 1e-5,
                       slots.to(gpu_device), cache, H, dn, dr, R)
    qr = proj[:, :H * (dn + dr)].view(T, H, dn + dr)[:, :, dn:]
    want_q = P.rotate_pairs(qr.double().transpose(0, 1), pos, 777.0, dims).transpose(0, 1).float() if dims else qr
    assert close(q[:, :, R:], want_q, 3e-4) and float(q[:, :, :R].abs().max()) == 0.0
    d = proj[:, H * (dn + dr):H * (dn + dr) + D]
    c = P.rms(d[:, :R], 1e-5) * cw
    kr = P.rotate_pairs(d[:, R:].double(), pos, 777.0, dims).float() if dims else d[:, R:]
    flat = cache.view(-1, D).cpu()
    for t in range(T):
        if slots[t] >= 0:
            assert close(flat[slots[t]][:R], c[t], 3e-6) and close(flat[slots[t]][R:], kr[t], 3e-4)
    untouched = [i for i in range(3 * page) if i not in slots.tolist()]
    assert torch.all(flat[untouched] == 9.0)


@pytest.mark.parametrize("dtype,K,N", [(torch.float32, 10, 36), (torch.bfloat16, 16, 48),
                                       (torch.bfloat16, 40, 70), (torch.bfloat16, 12, 20)],
                         ids=["fp32", "bf16-mfma", "bf16-mfma-tail", "bf16-fma"])
def test_per_head_products(gpu_device, dtype, K, N):
    from pytriton_llama_amd import ops
    T, H = 70, 5
    x = rnd(T, H, K + 8, seed=1).to(dtype)
    w = rnd(H, N, K, seed=2).to(dtype)
    gate = rnd(T, H + 3, seed=3).to(dtype)
    out = torch.zeros(T, H, N + 4, dtype=dtype, device=gpu_device)
    xd = x.to(gpu_device)
    ops.gemm_heads_nt(out[:, :, :N], xd[:, :, :K], w.to(gpu_device), gate.to(gpu_device)[:, 1:1 + H])
    want = torch.einsum("thk,hnk->thn", x[:, :, :K].float(), w.float())
    want = want * torch.sigmoid(gate[:, 1:1 + H].float())[:, :, None]
    assert close(out[:, :, :N], want, 1e-5 if dtype == torch.float32 else 1e-2)
    assert float(out[:, :, N:].abs().max()) == 0.0
    plain = torch.empty(T, H, N, dtype=dtype, device=gpu_device)
    ops.gemm_heads_nt(plain, xd[:, :, :K], w.to(gpu_device))
    assert close(plain, torch.einsum("thk,hnk->thn", x[:, :, :K].float(), w.float()),
                 1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("T,E,top,I,W", [(1, 4, 1, 24, 48), (7, 5, 2, 40, 48), (40, 2, 1, 24, 48),
                                          (150, 6, 3, 72, 48), (300, 70, 4, 16, 48), (260, 3, 2, 200, 48),
                                          (200, 4, 2, 192, 128), (333, 9, 3, 64, 64)])
def test_routed_experts(gpu_device, dtype, T, E, top, I, W):
    """Routing, grouping and the experts' products against a loop over tokens; the weight
    scales the expert's input (with the clamp in the activation that is not the same as
    scaling its output)."""
    from pytriton_llama_amd.parts import GatedMLP, RoutedExperts
    limit = 0.8
    tensors = {"router": rnd(E, W, seed=1, std=0.5), "shared.sg": rnd(1, W, seed=2, std=0.3)}
    for n, s in (("gate", 3), ("up", 4)):
        tensors["shared." + n] = rnd(32, W, seed=s, std=0.3)
    tensors["shared.down"] = rnd(W, 32, seed=5, std=0.3)
    for e in range(E):
        tensors[f"e{e}.gate"] = rnd(I, W, seed=10 + 3 * e, std=0.4)
        tensors[f"e{e}.up"] = rnd(I, W, seed=11 + 3 * e, std=0.4)
        tensors[f"e{e}.down"] = rnd(W, I, seed=12 + 3 * e, std=0.4)
    tensors = {k: v.to(dtype) for k, v in tensors.items()}
    part = RoutedExperts(W, I, E, top, "clamped", limit, True, False,
                         GatedMLP(W, 32, "clamped", 1.2), True)
    assert {s.name for s in part.param_sources()} == set(tensors)
    part.load(tensors, dtype, gpu_device)
    x = rnd(T, W, seed=99).to(dtype)
    got = part.forward(x.to(gpu_device))
    assert got.dtype == torch.float32
    Wf = {"m." + k: v.float() for k, v in tensors.items()}
    mlp = {"router": {"experts": E, "top": top}, "expert": {"limit": limit}, "shared": {"limit": 1.2}}
    want = P.moe_ff(x.float(), Wf, "m", mlp)
    assert close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)
    # every token went to its ``top`` best experts
    from pytriton_llama_amd import ops
    from pytriton_llama_amd.parts import linear
    r = ops.moe_route(linear(x.to(gpu_device), part.router, out_dtype=torch.float32), E, top, 1)
    z = x.float() @ tensors["router"].float().T
    assert torch.equal(r.idx.view(T, top).cpu().long().sort(-1).values, z.topk(top, -1).indices.sort(-1).values)
    assert torch.equal(r.sorted[r.pos_of.long()].cpu(), torch.arange(T * top, dtype=torch.int32))
    by_expert = r.idx[r.sorted.long()].cpu()
    assert torch.all(by_expert[1:] >= by_expert[:-1])


def test_clamped_activation_and_its_limit(gpu_device):
    from pytriton_llama_amd import ops
    gu = torch.tensor([[5.0, -5.0, 0.3, 5.0, -5.0, 0.2]])          # gate | up, I = 3
    got = ops.gated_act(gu.to(gpu_device), ops.ACT_CLAMPED, 2.0).cpu()
    g, u = torch.tensor([2.0, -5.0, 0.3]), torch.tensor([2.0, -2.0, 0.2])
    assert torch.allclose(got[0], g * torch.sigmoid(1.702 * g) * (u + 1), rtol=1e-6)
    got = ops.gated_act(gu.to(gpu_device), ops.ACT_SILU).cpu()
    assert torch.allclose(got[0], gu[0, :3] * torch.sigmoid(gu[0, :3]) * gu[0, 3:], rtol=1e-6)

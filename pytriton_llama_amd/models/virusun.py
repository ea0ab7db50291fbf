"""``Virusun``: layers given as a list, each with one of three mixers (differential attention that
may read another layer's keys and values; rotary attention and a matrix memory side by side; the
gated delta rule) and a dense feed-forward or none, an RMS norm on every sublayer's output, on a
float32 residual stream. The model is a list of layer specs over the engine's parts; tensor names
are the checkpoint's own ("l<i>.mix.q", "l<i>.mix.left.q", "l<i>.norm1", ...).
"""
from __future__ import annotations

from ..config.registry import register_model
from ..config.virusun_config import VirusunConfig
from ..parts.base import build_part
from .causal_lm import CausalLM, LayerCall

# role of a part inside a block -> what follows "l<i>." in its tensors' names
VIRUSUN_BLOCK_PREFIXES = {"norm1": "norm1", "norm2": "norm2", "mixer": "mix.", "feed_forward": "mlp."}


def _norm(cfg: VirusunConfig):
    return build_part("norm", "rmsnorm", size=cfg.hidden_size, eps=cfg.norm_eps, weight_name="")


def _mixer(cfg: VirusunConfig, layer):
    W, eps, m = cfg.hidden_size, cfg.norm_eps, layer.mixer
    if layer.kind == "attention":
        return build_part("mixer", "normed_attention", hidden_size=W, num_heads=m.heads, num_kv_heads=m.kv_heads,
                          dim=m.dim, vdim=m.vdim, scale=m.scale, eps=eps, qk_norm="head", maps=2, diff=m.diff,
                          bias=True, gated=True, own_kv=m.kv_from is None)
    if layer.kind == "parallel":
        l, r = m.left, m.right
        left = build_part("mixer", "normed_attention", hidden_size=W, num_heads=l.heads, num_kv_heads=l.kv_heads,
                          dim=l.dim, vdim=l.vdim, scale=l.scale, eps=eps, qk_norm="whole", maps=1, bias=True,
                          gated=False, rot_dims=l.rot.dims, rot_base=l.rot.base, rot_scaling=l.rot.scaling_dict())
        right = build_part("mixer", "matrix_memory", hidden_size=W, num_heads=r.heads, dim=r.dim, vdim=r.vdim,
                           gate_cap=r.gate_cap, eps=eps)
        return build_part("mixer", "parallel", left=left, right=right, left_scale=m.left_scale,
                          right_scale=m.right_scale)
    return build_part("mixer", "gated_delta", hidden_size=W, num_heads=m.heads, num_kv_heads=m.kv_heads,
                      dim=m.dim, vdim=m.vdim, taps=m.conv, eps=eps)


def build_virusun(cfg: VirusunConfig) -> CausalLM:
    W = cfg.hidden_size
    embedding = build_part("embedding", "token_embedding", vocab_size=cfg.vocab_size, hidden_size=W,
                           weight_name="embed", float32_stream=True)
    blocks, cache_layers, schedule = [], [], []
    cache_of = {}

    def keep(spec):
        if spec is None:
            return None
        cache_layers.append(spec)
        return len(cache_layers) - 1

    for i, layer in enumerate(cfg.layers):
        mixer = _mixer(cfg, layer)
        ffn = None
        if layer.ff:
            ffn = build_part("feed_forward", "swiglu", hidden_size=W, intermediate_size=layer.ff,
                             gate_name="gate", up_name="up", down_name="down")
        blocks.append(build_part("block", "output_norm", mixer=mixer, mixer_norm=_norm(cfg), feed_forward=ffn,
                                 ffn_norm=_norm(cfg) if ffn is not None else None))
        if layer.kind == "attention" and layer.mixer.kv_from is not None:
            schedule.append(LayerCall(i, cache_of[layer.mixer.kv_from], False))
            continue
        spec = mixer.cache_spec()
        cache_of[i] = tuple(keep(s) for s in spec) if isinstance(spec, tuple) else keep(spec)
        schedule.append(LayerCall(i, cache_of[i], True))
    blocks[-1].last = True                  # (the run order is the order of the layers)
    final_norm = _norm(cfg)
    head = build_part("head", "linear_head", vocab_size=cfg.vocab_size, hidden_size=W, weight_name="head")
    prefixes = [("", embedding)]
    for i, b in enumerate(blocks):
        for role, part in b.children().items():
            prefixes.append((f"l{i}.{VIRUSUN_BLOCK_PREFIXES[role]}", part))
    prefixes += [("final.norm", final_norm), ("", head)]
    return CausalLM(cfg, embedding, blocks, final_norm, head, cache_layers, schedule, prefixes)


register_model("Virusun", VirusunConfig, build_virusun)

"""``Rubasun``: latent-attention layers with Dynamic-Tanh norms in front of and behind every
sublayer, dense or routed feed-forwards, a scaled embedding and a gated per-layer token input,
on a float32 residual stream. The model is a list of layer specs over the engine's parts;
tensor names are the checkpoint's own ("l<i>.mix.q", "l<i>.norm1", "l<i>.norm1.alpha", ...).
A layer with ``kv_from`` keeps no cache: the run order hands it the owner's cache layer to read.
"""
from __future__ import annotations

from ..config.registry import register_model
from ..config.rubasun_config import RubasunConfig
from ..parts.base import build_part
from .causal_lm import CausalLM, LayerCall

# role of a part inside a block -> what follows "l<i>." in its tensors' names
RUBASUN_BLOCK_PREFIXES = {"norm1": "norm1", "norm1b": "norm1b", "norm2": "norm2", "norm2b": "norm2b",
                          "mixer": "mix.", "feed_forward": "mlp.", "side": "side."}


def _norm(cfg: RubasunConfig):
    # "<name>" is the weight itself, "<name>.b" and "<name>.alpha" lie beside it
    return build_part("norm", "dynamic_tanh", size=cfg.hidden_size, weight_name="", bias_name=".b",
                      alpha_name=".alpha")


def _feed_forward(cfg: RubasunConfig, mlp):
    W = cfg.hidden_size
    if mlp.kind == "dense":
        return build_part("feed_forward", "swiglu", hidden_size=W, intermediate_size=mlp.ff,
                          gate_name="gate", up_name="up", down_name="down")
    shared = None
    if mlp.shared is not None:
        shared = build_part("feed_forward", "gated_mlp", hidden_size=W, intermediate_size=mlp.shared.ff,
                            activation="clamped", limit=mlp.shared.limit)
    return build_part("feed_forward", "routed_experts", hidden_size=W, intermediate_size=mlp.expert.ff,
                      num_experts=mlp.experts, top=mlp.top, activation="clamped", limit=mlp.expert.limit,
                      weight_on_input=True, renormalize=False, shared=shared, shared_gate=True)


def build_rubasun(cfg: RubasunConfig) -> CausalLM:
    W = cfg.hidden_size
    embedding = build_part("embedding", "token_embedding", vocab_size=cfg.vocab_size, hidden_size=W,
                           weight_name="embed", scale=cfg.embedding_scale, float32_stream=True)
    table = None
    if cfg.token_side_dim:
        table = build_part("embedding", "token_table", vocab_size=cfg.vocab_size,
                           columns=len(cfg.layers) * cfg.token_side_dim, weight_name="embed")
    blocks, cache_layers, schedule = [], [], []
    cache_of = {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        mixer = build_part("mixer", "latent_attention", hidden_size=W, num_heads=m.heads, dim=m.dim,
                           rot_dim=m.rot_dim, vdim=m.vdim, kv_rank=m.kv_rank, scale=m.scale,
                           rot_base=m.rot_base, rot_dims=m.rot_dims, eps=cfg.norm_eps,
                           own_kv=m.kv_from is None, gated=True)
        ffn = _feed_forward(cfg, layer.mlp) if layer.mlp is not None else None
        side = None
        if table is not None:
            side = build_part("stream_input", "gated_token_input", hidden_size=W, dim=cfg.token_side_dim,
                              table=table, first_column=i * cfg.token_side_dim, eps=cfg.norm_eps)
        blocks.append(build_part("block", "sandwich", pre_mixer_norm=_norm(cfg), mixer=mixer,
                                 post_mixer_norm=_norm(cfg),
                                 pre_ffn_norm=_norm(cfg) if ffn is not None else None, feed_forward=ffn,
                                 post_ffn_norm=_norm(cfg) if ffn is not None else None, side=side))
        if m.kv_from is None:
            cache_of[i] = len(cache_layers)
            cache_layers.append(mixer.cache_spec())
            schedule.append(LayerCall(i, cache_of[i], True))
        else:
            schedule.append(LayerCall(i, cache_of[m.kv_from], False))
    for before, after in zip(blocks, blocks[1:]):      # (the run order is the order of the layers)
        before.next_norm = after.norm1
    final_norm = _norm(cfg)
    head = build_part("head", "linear_head", vocab_size=cfg.vocab_size, hidden_size=W, weight_name="head")
    prefixes = [("", embedding)]
    if table is not None:
        prefixes.append(("side.", table))
    for i, b in enumerate(blocks):
        for role, part in b.children().items():
            prefixes.append((f"l{i}.{RUBASUN_BLOCK_PREFIXES[role]}", part))
    prefixes += [("final.norm", final_norm), ("", head)]
    return CausalLM(cfg, embedding, blocks, final_norm, head, cache_layers, schedule, prefixes)


register_model("Rubasun", RubasunConfig, build_rubasun)

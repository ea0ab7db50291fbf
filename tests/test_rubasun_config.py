"""Rubasun's configuration and model assembly (no GPU)."""
import pytest
import torch

import pytriton_llama_amd  # noqa: F401
from pytriton_llama_amd.config import ConfigError, build_model, config_from_dict
from pytriton_llama_amd.models import LayerCall
from rubasun_configs import rubasun


def test_every_size_comes_from_the_file():
    cfg, _, _ = rubasun("R1")
    c = config_from_dict(cfg)
    assert (c.vocab_size, c.hidden_size, c.embedding_scale, c.norm_eps, c.token_side_dim) == (200, 64, 6.0, 1e-5, 8)
    assert [l.mixer.kv_from for l in c.layers] == [None, None, 1, 1, None]
    assert [None if l.mlp is None else l.mlp.kind for l in c.layers] == ["dense", "moe", "moe", None, "dense"]
    assert c.layers[1].mlp.shared.ff == 56 and c.layers[2].mlp.shared is None
    for key in ("vocab", "width", "layers", "embedding", "norm"):
        bad = dict(cfg)
        del bad[key]
        with pytest.raises(ConfigError):
            config_from_dict(bad)


def test_a_layer_may_only_read_an_earlier_cache_of_equal_shape():
    cfg, _, _ = rubasun("R1")
    cfg["layers"][2]["mixer"]["kv_from"] = 3
    with pytest.raises(ConfigError):
        config_from_dict(cfg)
    cfg, _, _ = rubasun("R1")
    cfg["layers"][3]["mixer"]["kv_from"] = 2          # layer 2 has no cache of its own
    with pytest.raises(ConfigError):
        config_from_dict(cfg)
    cfg, _, _ = rubasun("R1")
    cfg["layers"][2]["mixer"]["kv_rank"] = 32
    with pytest.raises(ConfigError):
        config_from_dict(cfg)
    cfg, _, _ = rubasun("R1")
    cfg["layers"][0]["type"] = "something_else"
    with pytest.raises(ConfigError):
        config_from_dict(cfg)


def test_run_order_and_tensor_names():
    cfg, _, _ = rubasun("R1")
    m = build_model(cfg)
    assert m.schedule == [LayerCall(0, 0, True), LayerCall(1, 1, True), LayerCall(2, 1, False),
                          LayerCall(3, 1, False), LayerCall(4, 2, True)]
    assert len(m.cache_layers) == 3 and len({repr(s) for s in m.cache_layers}) == 1
    names = m.expected_tensors()
    for n, shape in {"embed": (200, 64), "side.embed": (200, 40), "l0.norm1": (64,), "l0.norm1.alpha": (),
                     "l0.norm2b.b": (64,), "l0.mix.q": (128, 64), "l0.mix.dkv": (64, 64),
                     "l0.mix.dkv.norm": (48,), "l0.mix.uk": (64, 48), "l0.mix.uv": (96, 48),
                     "l0.mix.g": (4, 64), "l0.mix.o": (64, 96), "l0.mlp.gate": (96, 64),
                     "l1.mlp.router": (5, 64), "l1.mlp.e4.down": (64, 40), "l1.mlp.shared.up": (56, 64),
                     "l1.mlp.shared.sg": (1, 64), "l3.side.proj": (64, 8), "final.norm.b": (64,),
                     "head": (200, 64)}.items():
        assert tuple(names[n][1].shape) == shape, n
    for absent in ("l2.mix.dkv", "l2.mix.dkv.norm", "l2.mlp.shared.gate", "l3.norm2", "l3.mlp.gate"):
        assert absent not in names
    cfg2, _, _ = rubasun("R2")
    assert "side.embed" not in build_model(cfg2).expected_tensors()


def test_random_model_folder_round_trip(tmp_path):
    from pytriton_llama_amd.weights import write_random_model
    from safetensors.torch import load_file
    cfg, std, _ = rubasun("R4")
    folder = write_random_model(cfg, str(tmp_path), seed=3, dtype=torch.float32, std=std, norm_std=0.1)
    w = load_file(str(tmp_path / "model.safetensors"))
    assert set(w) == set(build_model(cfg).expected_tensors())
    assert w["l0.norm1.alpha"].shape == () and 0.3 < float(w["l0.norm1.alpha"]) < 1.3

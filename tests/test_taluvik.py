"""The Taluvik architecture without a GPU: its configuration, the model it describes, tensor names,
cache needs, and the plain implementation's own consistency."""

import copy
import json

import pytest
import torch

from . import taluvik_models as models
from .helpers import random_tokens
from .plain import taluvik as plain


def test_config_round_trip_and_registry(tmp_path):
    from torchllms_amd.config import TaluvikConfig, architecture_of, load_config

    for name, raw in models.CONFIGS.items():
        cfg = TaluvikConfig.from_dict(raw)
        assert TaluvikConfig.from_dict(cfg.to_dict()) == cfg
        assert architecture_of(cfg).name == "Taluvik"
        (tmp_path / name).mkdir()
        with open(tmp_path / name / "config.json", "w") as f:
            json.dump(raw, f)
        arch, again = load_config(tmp_path / name)
        assert arch.name == "Taluvik" and again == cfg


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].__setitem__("type", "lstm"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("softcap"), "softcap"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("heads", 3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 34), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "dense"),
    (lambda c: c["layers"][3].__setitem__("weights_of", 3), "weights_of"),
    (lambda c: c["layers"][3].__setitem__("weights_of", 17), "weights_of"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["layers"][2]["mixer"].__setitem__("state", 0), "state"),
])
def test_config_refuses(change, message):
    from torchllms_amd.config import ConfigError, TaluvikConfig

    raw = copy.deepcopy(models.CONFIG_A)
    change(raw)
    with pytest.raises(ConfigError, match=message):
        TaluvikConfig.from_dict(raw)


def test_layers_that_borrow_tensors_run_their_owner_again():
    from torchllms_amd.config import TaluvikConfig, taluvik_model_spec
    from torchllms_amd.parts import KVNeed, Model, StateNeed

    cfg = TaluvikConfig.from_dict(models.CONFIG_A)
    spec = taluvik_model_spec(cfg)
    assert [l.name for l in spec.layers] == ["l0", "l1", "l2", "l5"]
    assert [r.layer for r in spec.order] == [0, 1, 2, 0, 2, 3] and all(r.cache_from is None for r in spec.order)
    assert spec.layers[3].block == "parallel_mixer" and spec.layers[0].block == "parallel"
    model = Model(spec)
    needs = dict(model.cache_needs())
    assert len(needs) == 6  # a cache entry or a state for every run, shared tensors or not
    assert needs[(0, "mix")] == needs[(3, "mix")] == KVNeed(num_kv_heads=2, head_dim=32, v_head_dim=16)
    taps, c = 4, 2 * 2 * 16 + 4 * 32
    assert needs[(1, "mix")] == StateNeed(shape=((taps - 1) * c + 4 * 32 * 16,))
    assert needs[(2, "mix")] == needs[(4, "mix")] == StateNeed(shape=(3 * 96 + 96 * 16,))
    names = set(model.param_specs())
    assert "l0.mix.sinks" in names and "l3.mix.wq.weight" not in names and "l5.mlp.w1.weight" not in names


def test_keys_and_values_of_different_head_sizes_get_pages_of_their_own_shape():
    from torchllms_amd.cache.manager import CacheManager, group_layers
    from torchllms_amd.parts import KVNeed

    groups, states = group_layers([("a", KVNeed(2, 32, v_head_dim=16)), ("b", KVNeed(2, 32, v_head_dim=16)),
                                   ("c", KVNeed(2, 32)), ("d", KVNeed(2, 32, v_head_dim=32))])
    assert [g.run_ids for g in groups] == [("a", "b"), ("c", "d")] and not states
    assert [g.value_dim for g in groups] == [16, 32]
    assert CacheManager.bytes_per_token(groups, torch.bfloat16) == 2 * (2 * 2 * 48 + 2 * 2 * 64)
    cache = CacheManager(groups, states, page_size=4, num_pages=3, max_seqs=2, dtype=torch.float32, device="cpu")
    assert cache.k_pages[0].shape == (2, 3, 2, 4, 32) and cache.v_pages[0].shape == (2, 3, 2, 4, 16)
    assert cache.kv_view("b").v_pages.shape == (3, 2, 4, 16)


def test_model_folder_round_trip_through_the_loader(tmp_path):
    from torchllms_amd.config import load_config
    from torchllms_amd.parts import Model
    from torchllms_amd.weights import load_weights

    folder = models.make_folder(tmp_path / "m", models.CONFIG_B, seed=1)
    raw, tensors = models.read_folder(folder)
    assert raw["architecture"] == "Taluvik" and "l3.mix.q" not in tensors and "l1.mix.q.conv" in tensors
    arch, cfg = load_config(folder)
    model = Model(arch.model_spec(cfg))
    loaded = load_weights(folder, arch.weight_rules(cfg), model.param_specs(), torch.float32)
    assert set(loaded) == set(model.param_specs())
    assert torch.equal(loaded["l2.mix.sinks"], tensors["l2.mix.sink"].float())
    assert torch.equal(loaded["final_norm.bias"], tensors["final.norm.b"].float())


# ----------------------------------------------------------------------------- the plain implementation against itself
def _weights(raw, seed, tmp_path):
    folder = models.make_folder(tmp_path / f"w{seed}", raw, seed=seed)
    cfg, tensors = models.read_folder(folder)
    return cfg, {k: v.double() for k, v in tensors.items()}


def test_plain_attention_sees_its_chunk_and_nothing_else():
    g = torch.Generator().manual_seed(0)
    S, d, dv, chunk = 40, 8, 4, 16
    q, k, v = (torch.randn((S, n), generator=g, dtype=torch.float64) for n in (d, d, dv))
    pos = torch.arange(S)
    sink = torch.tensor(0.3, dtype=torch.float64)
    out = plain.attention_scores_to_output(q, k, v, 0.5, 10.0, chunk, sink, pos)
    # one row by hand
    i = 37
    s = 10.0 * torch.tanh((k[32 : i + 1] @ q[i]) * 0.5 / 10.0)
    p = torch.exp(s) / (torch.exp(s).sum() + torch.exp(sink))
    assert torch.allclose(out[i], p @ v[32 : i + 1], atol=1e-12)
    # a chunk's first position sees itself alone: its value scaled down by the sink's share
    s0 = 10.0 * torch.tanh((k[16] @ q[16]) * 0.5 / 10.0)
    assert torch.allclose(out[16], v[16] * torch.exp(s0) / (torch.exp(s0) + torch.exp(sink)), atol=1e-12)
    # keys of other chunks change nothing
    k2, v2 = k.clone(), v.clone()
    k2[:32] += 5.0
    v2[:32] -= 3.0
    assert torch.equal(plain.attention_scores_to_output(q, k2, v2, 0.5, 10.0, chunk, sink, pos)[32:], out[32:])
    # the same rows come out when the sequence is handed over from position 32 on
    tail = plain.attention_scores_to_output(q[32:], k[32:], v[32:], 0.5, 10.0, chunk, sink, pos[32:])
    assert torch.allclose(tail, out[32:], atol=1e-12)


def test_plain_rotation_pairs_halves_and_scales_long_waves():
    freqs = plain.rotary_frequencies(8, 100.0, None)
    assert freqs == [100.0 ** (-2 * i / 8) for i in range(4)]
    scaled = plain.rotary_frequencies(8, 100.0, {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 16})
    # wavelengths 6.3, 19.9, 62.8, 198.7 against the band 4 .. 16: the first lies in the band, the others beyond it
    assert scaled[1:] == [f / 4.0 for f in freqs[1:]]
    s = (16 / (2 * torch.pi) - 1.0) / 3.0
    assert abs(scaled[0] - ((1 - s) / 4.0 + s)) < 1e-12
    x = torch.zeros((1, 1, 6), dtype=torch.float64)
    x[0, 0, 0], x[0, 0, 4] = 1.0, 7.0
    out = plain.rotate(x, torch.tensor([3]), [0.5, 0.25], 4)
    assert torch.allclose(out[0, 0], torch.tensor([torch.cos(torch.tensor(1.5)), 0, torch.sin(torch.tensor(1.5)), 0, 7.0, 0], dtype=torch.float64))


def test_plain_recurrences_carry_what_a_cut_would_lose(tmp_path):
    """The weights of the tests make a lost state, a forgotten sink and a chunk that is one token off
    visible in the logits: far above the tolerance that the engine is held to."""
    cfg, w = _weights(models.CONFIG_A, 3, tmp_path)
    toks = random_tokens(90, cfg["vocab"], 5)
    base = plain.forward(cfg, w, toks)

    def rel(other):
        return float((other - base).std() / base.std())

    assert rel(plain.forward(cfg, {k: (v * 0 - 30 if k.endswith("sink") else v) for k, v in w.items()}, toks)) > 1e-2
    moved = copy.deepcopy(cfg)
    for layer in moved["layers"]:
        if layer["type"] == "attention":
            layer["mixer"]["mask"]["size"] += 1
    assert rel(plain.forward(moved, w, toks)) > 1e-2
    for i, layer in enumerate(cfg["layers"]):
        if "weights_of" not in layer:
            off = dict(w)
            off[f"l{i}.mix.o"] = w[f"l{i}.mix.o"] * 0
            assert rel(plain.forward(cfg, off, toks)) > 1e-2
    tail = plain.forward(cfg, w, toks[50:])
    assert float((tail[-1] - base[-1]).std() / base.std()) > 1e-2


def test_plain_convolution_and_layers():
    x = torch.arange(12, dtype=torch.float64).reshape(6, 2)
    taps = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 2.0]], dtype=torch.float64)
    out = plain.causal_conv(x, taps, torch.tensor([0.5, 0.0], dtype=torch.float64))
    assert out[0].tolist() == [0.5, 2.0] and out[1].tolist() == [200.5, 6.0] and out[3].tolist() == [600 + 40 + 2 + 0.5, 14.0]
    h = torch.randn((5, 7), dtype=torch.float64)
    ln = plain.layer_norm(h, torch.ones(7, dtype=torch.float64), torch.zeros(7, dtype=torch.float64), 0.0)
    assert torch.allclose(ln.mean(-1), torch.zeros(5, dtype=torch.float64), atol=1e-12)
    assert torch.allclose((ln ** 2).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-12)

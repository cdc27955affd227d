"""Vobolorn without a GPU: configuration, the model as data, tensor names, what the cache keeps, and the plain
implementation pinned against rows worked out by hand; and that the tests' weights make every mechanism show."""

import copy
import math

import pytest
import torch

from . import vobolorn_models as models
from .helpers import random_tokens
from .plain import vobolorn as plain


def _config(d):
    from torchllms_amd.config.vobolorn import VobolornConfig

    return VobolornConfig.from_dict(d)


# ----------------------------------------------------------------------------- configuration
def test_configuration_reads_every_size_and_writes_it_back():
    from torchllms_amd.config.registry import architecture_name, get_architecture

    for d in models.CONFIGS.values():
        cfg = _config(d)
        assert architecture_name(cfg.to_dict()) == "Vobolorn"
        assert _config(cfg.to_dict()) == cfg
        arch = get_architecture("Vobolorn")
        assert arch.config_from_dict(arch.config_json(cfg)) == cfg
    a = _config(models.CONFIG_A)
    assert (a.vocab, a.width, a.norm_eps, a.logit_softcap) == (131, 64, 1e-5, 12.0)
    assert [l.type for l in a.layers] == ["attention_2", "latent_attention", "attention", "attention_2"]
    assert a.layers[3].ff is None and a.layers[1].ff == 48
    assert a.first_mixing_layer() == 0 and _config(models.CONFIG_B).first_mixing_layer() == 2
    assert _config(models.CONFIG_B).logit_softcap == 0.0


@pytest.mark.parametrize("change, says", [
    (lambda d: d.pop("vocab"), "vocab"),
    (lambda d: d["norm"].update(eps=0), "eps"),
    (lambda d: d.update(logit_softcap=-1.0), "logit_softcap"),
    (lambda d: d["layers"][0].update(type="attention_3"), "type"),
    (lambda d: d["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda d: d["layers"][0]["mixer"].pop("q_temp"), "q_temp"),
    (lambda d: d["layers"][0]["mixer"]["q_temp"].update(every=0), "every"),
    (lambda d: d["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda d: d["layers"][1]["mixer"].update(rot_dim=7), "rot"),
    (lambda d: d["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda d: d["layers"][2]["mixer"].update(vdim=24), "v_mix"),
    (lambda d: d["layers"][0]["mlp"].update(kind="routed"), "dense"),
    (lambda d: d.update(layers=[]), "layers"),
])
def test_configuration_errors_name_what_is_wrong(change, says):
    from torchllms_amd.config.llama import ConfigError

    d = copy.deepcopy(models.CONFIG_A)
    change(d)
    with pytest.raises(ConfigError, match=says):
        _config(d)


# ----------------------------------------------------------------------------- the model as data
def test_the_model_is_made_of_registered_parts():
    from torchllms_amd.config.vobolorn import vobolorn_model_spec
    from torchllms_amd.parts.attention import Attention
    from torchllms_amd.parts.latent import LatentAttention
    from torchllms_amd.parts.model import Model

    model = Model(vobolorn_model_spec(_config(models.CONFIG_A)))
    kinds = [type(b).__name__ for b in model.blocks]
    assert kinds == ["BranchNormBlock", "BranchNormBlock", "BranchNormBlock", "BranchNormMixerBlock"]
    mixers = [b.mix for b in model.blocks]
    assert isinstance(mixers[1], LatentAttention) and all(isinstance(mixers[i], Attention) for i in (0, 2, 3))
    assert [m.value_mix for m in (mixers[0], mixers[2], mixers[3])] == ["source", "mix", "mix"]
    assert (mixers[0].q_temp_coef, mixers[0].q_temp_every, mixers[3].q_temp_every) == (0.5, 7, 16)
    assert mixers[2].qkv_bias and mixers[2].out_gate == "channel" and not mixers[0].qkv_bias and mixers[0].out_gate is None
    assert all(m.prepared and m.qk_norm_weight for m in (mixers[0], mixers[2], mixers[3]))
    assert model.head.softcap == 12.0 and model.embedding.stream_dtype == "float32"
    assert all(p.graph_safe for p in model.all_parts())
    specs = model.param_specs()
    assert specs["l2.mix.vmix"].shape == () and "l0.mix.vmix" not in specs and "l0.mix.vmix" in model.ignorable_tensors()
    assert specs["l2.mix.wg.weight"].shape == (4 * 16, 64) and specs["l1.mix.wg.weight"].shape == (3, 64)
    assert specs["l1.mix.dkv.weight"].shape == (40 + 8, 64) and specs["l1.mix.uq.weight"].shape == (3 * (24 + 8), 28)
    assert specs["l2.mix.wv.bias"].shape == (2 * 16,) and specs["l2.mix.q_norm.weight"].shape == (24,)
    assert "l3.norm2.weight" not in specs and "l3.mlp.w1.weight" not in specs


def test_every_tensor_has_a_checkpoint_name_and_comes_back(tmp_path):
    from torchllms_amd.config.registry import load_config
    from torchllms_amd.parts.model import Model
    from torchllms_amd.weights.loader import load_weights

    folder = models.make_folder(tmp_path / "m", models.CONFIG_A, seed=3)
    _, tensors = models.read_folder(folder)
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.q.norm", "l2.mix.q.b", "l2.mix.vmix", "l2.mix.g",
            "l1.mix.dkv.norm", "l1.mix.uk", "l3.mix.o", "l0.mlp.gate"} <= set(tensors)
    assert "l3.norm2" not in tensors and "l0.mix.q.b" not in tensors
    arch, cfg = load_config(folder)
    model = Model(arch.model_spec(cfg))
    loaded = load_weights(folder, arch.weight_rules(cfg), model.param_specs(), torch.float32)
    assert set(loaded) == set(model.param_specs())
    assert torch.equal(loaded["l2.mix.wq.bias"], tensors["l2.mix.q.b"].float())
    assert 0.25 <= float(loaded["l2.mix.vmix"]) <= 0.75
    # a checkpoint may carry the first mixing layer's unused factor
    from safetensors.torch import save_file

    tensors["l0.mix.vmix"] = torch.tensor(0.5, dtype=torch.bfloat16)
    save_file(tensors, str(folder / "model.safetensors"))
    with pytest.warns(UserWarning, match="l0.mix.vmix"):
        load_weights(folder, arch.weight_rules(cfg), model.param_specs(), torch.float32, ignore_when_present=model.ignorable_tensors())


def test_the_cache_keeps_one_row_per_token_for_a_latent_layer():
    from torchllms_amd.cache.manager import CacheManager, group_layers
    from torchllms_amd.config.vobolorn import vobolorn_model_spec
    from torchllms_amd.parts.model import Model

    model = Model(vobolorn_model_spec(_config(models.CONFIG_A)))
    needs = dict(model.cache_needs())
    latent = needs[(1, "mix")]
    assert (latent.num_kv_heads, latent.head_dim, latent.v_head_dim, latent.values_in_keys) == (1, 48, 40, True)
    assert (needs[(0, "mix")].head_dim, needs[(0, "mix")].v_head_dim) == (32, 16)
    groups, states = group_layers(model.cache_needs())
    assert not states and len(groups) == 4  # three sizes of grouped-query layers and the latent one
    by_run = {g.run_ids: g for g in groups}
    assert by_run[((1, "mix"),)].elements_per_token == 48
    assert by_run[((0, "mix"),)].elements_per_token == 2 * (32 + 16)
    total = 2 * (32 + 16) + 48 + 2 * (24 + 16) + 2 * (40 + 16)
    assert CacheManager.bytes_per_token(groups, torch.bfloat16) == 2 * total


# ----------------------------------------------------------------------------- the plain implementation, by hand
def test_the_query_factor_steps_with_the_floor():
    f = plain.query_temperature(13, 0.5, 4, torch.float64)
    assert f[0] == f[2] == 1.0                                   # floor(1/4) .. floor(3/4) = 0
    assert f[3] == f[6] == 1.0 + 0.5 * math.log(2.0)             # positions 3..6: floor((p + 1) / 4) = 1
    assert f[7] == 1.0 + 0.5 * math.log(3.0) and f[11] == 1.0 + 0.5 * math.log(4.0)
    every_token = plain.query_temperature(3, 1.0, 1, torch.float64)
    assert torch.allclose(every_token, torch.tensor([1 + math.log(2), 1 + math.log(3), 1 + math.log(4)], dtype=torch.float64))


def test_rotation_turns_neighbouring_channels_and_passes_the_rest():
    x = torch.zeros((3, 1, 6), dtype=torch.float64)
    x[:, 0] = torch.tensor([1.0, 0.0, 0.0, 2.0, 5.0, 7.0])
    y = plain.rotate_pairs(x, 100.0, 4)
    assert torch.equal(y[0], x[0])                               # position 0: no turn
    a0, a1 = 2.0, 2.0 * 100.0 ** -0.5                            # angles of the two pairs at position 2
    want = torch.tensor([math.cos(a0), math.sin(a0), -2.0 * math.sin(a1), 2.0 * math.cos(a1), 5.0, 7.0], dtype=torch.float64)
    assert torch.allclose(y[2, 0], want)


def test_the_norm_has_eps_under_the_root_and_a_plain_weight():
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    w = torch.tensor([2.0, 0.5], dtype=torch.float64)
    assert torch.allclose(plain.rms_norm(x, w, 0.5), torch.tensor([[3.0 * 2.0, 4.0 * 0.5]], dtype=torch.float64) / math.sqrt(12.5 + 0.5))


def test_scores_against_the_latent_are_the_scores_against_expanded_keys():
    """What the engine's latent layer rests on: with q' = W_uk[h]^T q the score q . (W_uk[h] c) is q' . c, and
    W_uv[h] applied to the mixed latents is the mix of the expanded values."""
    g = torch.Generator().manual_seed(0)
    S, H, d, r, dv, R = 9, 3, 5, 4, 6, 7
    q = torch.randn((S, H, d + r), generator=g, dtype=torch.float64)
    c = torch.randn((S, R), generator=g, dtype=torch.float64)
    k_rot = torch.randn((S, 1, r), generator=g, dtype=torch.float64)
    w_uk = torch.randn((H * d, R), generator=g, dtype=torch.float64)
    w_uv = torch.randn((H * dv, R), generator=g, dtype=torch.float64)
    keys = torch.cat([(c @ w_uk.T).reshape(S, H, d), k_rot.expand(S, H, r)], dim=-1)
    want = plain.causal_softmax_attention(q, keys, (c @ w_uv.T).reshape(S, H, dv), 0.3)
    q_lat = torch.einsum("shd,hdr->shr", q[..., :d], w_uk.reshape(H, d, R))
    rows = torch.cat([c, k_rot[:, 0]], dim=-1).reshape(S, 1, R + r)
    mixed = plain.causal_softmax_attention(torch.cat([q_lat, q[..., d:]], dim=-1), rows, c.reshape(S, 1, R), 0.3)
    got = torch.einsum("shr,hvr->shv", mixed, w_uv.reshape(H, dv, R))
    assert torch.allclose(got, want, atol=1e-12)


def test_the_tests_weights_make_every_mechanism_show(tmp_path):
    """Taking any one mechanism out of the plain model moves the logits by far more than the tests' 32-bit bound,
    so the comparison with the engine would see it missing."""
    folder = models.make_folder(tmp_path / "m", models.CONFIG_A, seed=11)
    cfg, weights = models.read_folder(folder)
    w = {k: v.double() for k, v in weights.items()}
    tokens = random_tokens(60, cfg["vocab"], 1)
    truth = plain.forward(cfg, w, tokens)
    scale = float((truth - truth.mean(-1, keepdim=True)).pow(2).mean().sqrt())

    def moved(config=None, tensors=None):
        z = plain.forward(config or cfg, tensors or w, tokens)
        d = z - truth
        d = d - d.mean(-1, keepdim=True)
        return float(d.pow(2).mean(-1).sqrt().max()) / scale

    def without(path, value):
        c = copy.deepcopy(cfg)
        node = c
        for key in path[:-1]:
            node = node[key]
        if value is None:
            node.pop(path[-1])
        else:
            node[path[-1]] = value
        return c

    def changed(name, fn):
        t = dict(w)
        t[name] = fn(w[name])
        return t

    bound = 100 * 2e-5
    assert moved(without(["logit_softcap"], None)) > bound
    assert moved(without(["layers", 0, "mixer", "q_temp", "coef"], 0.0)) > bound
    assert moved(without(["layers", 0, "mixer", "q_temp", "every"], 8)) > bound          # a step one token late
    assert moved(without(["layers", 2, "mixer", "v_mix"], False)) > bound
    assert moved(without(["layers", 3, "mixer", "v_mix"], False)) > bound
    assert moved(without(["layers", 1, "mixer", "rot", "base"], 9000.0)) > bound
    assert moved(tensors=changed("l2.mix.vmix", lambda t: 1.0 - t)) > bound
    assert moved(tensors=changed("l2.mix.q.b", torch.zeros_like)) > bound
    assert moved(tensors=changed("l2.mix.k.b", torch.zeros_like)) > bound
    assert moved(tensors=changed("l2.mix.v.b", torch.zeros_like)) > bound
    assert moved(tensors=changed("l2.mix.g", torch.zeros_like)) > bound
    assert moved(tensors=changed("l1.mix.g", torch.zeros_like)) > bound
    assert moved(tensors=changed("l0.mix.q.norm", torch.ones_like)) > bound
    assert moved(tensors=changed("l1.mix.dkv.norm", torch.ones_like)) > bound
    assert moved(tensors=changed("l1.mix.dq.norm", torch.ones_like)) > bound
    assert moved(tensors=changed("l3.norm1", torch.ones_like)) > bound
    # the rotated part of the latent layer's keys: without it the scores lose their only view of positions
    assert moved(tensors=changed("l1.mix.dkv", lambda t: torch.cat([t[:40], torch.zeros_like(t[40:])]))) > bound
    # a key far back: the first token's row of the embedding changed moves the last position's logits
    far = plain.forward(cfg, w, [(tokens[0] + 1) % cfg["vocab"]] + tokens[1:])
    d = far[-1] - truth[-1]
    assert float((d - d.mean()).pow(2).mean().sqrt()) / scale > bound

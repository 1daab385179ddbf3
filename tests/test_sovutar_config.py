"""Sovutar's configuration, recipe and cache needs (no GPU)."""
import copy

import pytest

from arle_amd.cache.manager import PagedNeed
from arle_amd.config import ConfigError, SovutarConfig, detect_architecture
from arle_amd.models.decoder import declared_cache_needs, expected_checkpoint_tensors, kv_cache_bytes_per_token
from tiny_sovutar import TINY

import torch


@pytest.mark.parametrize("name", list(TINY))
def test_a_configuration_reads_back_equal_and_names_its_tensors(name):
    raw = TINY[name][0]
    config = SovutarConfig.from_dict(raw)
    assert SovutarConfig.from_dict(config.to_dict()) == config
    arch = detect_architecture(raw)
    assert arch.name == "Sovutar"
    spec = arch.recipe(config, ())
    expected = expected_checkpoint_tensors(spec)
    assert expected["embed"].shape == (raw["vocab"], raw["width"]) and "final.norm" in expected and "head" in expected
    first = config.first_value_mixer()
    for i, layer in enumerate(raw["layers"]):
        m = layer["mixer"]
        if layer["type"] == "attention":
            assert expected[f"l{i}.mix.q.norm"].shape == (m["heads"] * m["dim"],)       # over the whole projection
            assert expected[f"l{i}.mix.k.norm"].shape == (m["kv_heads"] * m["dim"],)
            assert (f"l{i}.mix.vmix" in expected) == (bool(m.get("v_mix")) and i != first)
            if f"l{i}.mix.vmix" in expected:
                assert expected[f"l{i}.mix.vmix"].shape == ()
        else:
            assert expected[f"l{i}.mix.dkv"].shape == (m["kv_rank"] + m["rot_dim"], raw["width"])
            assert expected[f"l{i}.mix.uk"].shape == (m["heads"] * m["dim"], m["kv_rank"])
            assert expected[f"l{i}.mix.sink"].shape == (m["heads"],)
        if layer["mlp"] is None:
            assert f"l{i}.norm2" not in expected and f"l{i}.mlp.router" not in expected
        else:
            r = layer["mlp"]["router"]
            assert expected[f"l{i}.mlp.e{r['experts'] - 1}.down"].shape == (raw["width"], layer["mlp"]["expert"]["ff"])
            assert (f"l{i}.mlp.shared.gate" in expected) == (layer["mlp"]["shared"] is not None)


def test_the_cache_holds_one_latent_a_token_and_windows_give_pages_back():
    raw = TINY["P"][0]
    spec = detect_architecture(raw).recipe(SovutarConfig.from_dict(raw), ())
    needs = declared_cache_needs(spec)
    assert all(isinstance(n, PagedNeed) for n in needs)
    lat = raw["layers"][1]["mixer"]
    assert needs[1].window == lat["mask"]["size"] and needs[0].window is None
    assert needs[0].chunk == raw["layers"][0]["mixer"]["mask"]["size"] and needs[1].chunk is None
    shapes = {t.name: t.page_shape(4) for t in needs[1].page_tensors()}
    assert shapes == {"k": (1, 4, lat["kv_rank"] + lat["rot_dim"]), "v": (1, lat["kv_rank"], 4)}
    per_token = sum(2 * (l["mixer"]["kv_rank"] * 2 + l["mixer"]["rot_dim"]) if l["type"] == "latent_attention"
                    else 2 * l["mixer"]["kv_heads"] * (l["mixer"]["dim"] + l["mixer"]["vdim"]) for l in raw["layers"])
    assert kv_cache_bytes_per_token(spec, torch.bfloat16) == per_token


def broken(change):
    raw = copy.deepcopy(TINY["P"][0])
    change(raw)
    return raw


@pytest.mark.parametrize("change,word", [
    (lambda r: r["layers"][0].update(type="mamba"), "unknown layer type"),
    (lambda r: r["layers"][0]["mixer"].update(heads=5), "divisible"),
    (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda r: r["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda r: r["layers"][0]["mlp"].update(kind="dense"), "unknown kind"),
    (lambda r: r["layers"][0]["mlp"]["router"].update(top=9), "top"),
    (lambda r: r["layers"][2]["mixer"].update(vdim=8), "cannot be mixed"),
    (lambda r: r["layers"][0]["mixer"]["mask"].update(size=0), "mask.size"),
    (lambda r: r.update(layers=[]), "at least one layer"),
    (lambda r: r.pop("width"), "width"),
])
def test_a_configuration_that_cannot_be_used_is_refused_with_its_key(change, word):
    with pytest.raises(ConfigError) as exc:
        SovutarConfig.from_dict(broken(change))
    assert word in str(exc.value)


def test_a_model_without_a_cap_or_a_mask_is_taken():
    raw = broken(lambda r: (r.pop("logit_softcap"), r["layers"][0]["mixer"].pop("mask"), r["layers"][1]["mixer"].pop("mask")))
    config = SovutarConfig.from_dict(raw)
    assert config.logit_softcap == 0.0 and config.layers[0].mixer.chunk is None and config.layers[1].mixer.window is None
    raw = broken(lambda r: [l["mixer"].pop("kv_heads") for l in r["layers"] if l["type"] == "attention"])
    assert all(l.mixer.kv_heads == l.mixer.heads for l in SovutarConfig.from_dict(raw).layers if l.type == "attention")

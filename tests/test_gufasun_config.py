"""Gufasun on the CPU: configuration, recipe, and the cache manager's trees of named needs."""
import copy

import pytest
import torch

from arle_amd.cache import CacheManager, PagedNeed, StateNeed
from arle_amd.cache.manager import PagedView, StateView, need_leaves
from arle_amd.config import ConfigError, GufasunConfig, detect_architecture
from arle_amd.models import declared_cache_needs, expected_checkpoint_tensors
from tiny_gufasun import TINY_P, TINY_Q


def test_configuration_reads_back_and_names_its_design_with_one_string():
    for raw in (TINY_P, TINY_Q):
        c = GufasunConfig.from_dict(raw)
        assert GufasunConfig.from_dict(c.to_dict()) == c
        assert detect_architecture(c.to_dict()).name == "Gufasun"
    c = GufasunConfig.from_dict(TINY_P)
    assert (c.vocab, c.width, c.canon_taps, c.eps) == (211, 72, 3, 2e-5)
    assert c.layers[2].mixer.kv_from == 0 and c.layers[3].ff is None
    assert c.cache_window(0) == 21      # the reader's window is the wider one


@pytest.mark.parametrize("change, word", [
    (lambda r: r["layers"][2]["mixer"].update(kv_from=1), "kv_from"),           # an mLSTM layer has no keys
    (lambda r: r["layers"][2]["mixer"].update(kv_from=2), "kv_from"),           # not an earlier layer
    (lambda r: r["layers"][2]["mixer"].update(vdim=16), "differ"),
    (lambda r: r["layers"][0].update(type="conv"), "unknown layer type"),
    (lambda r: r["layers"][1]["mlp"].update(kind="moe"), "unknown kind"),
    (lambda r: r["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda r: r["layers"][0]["mixer"].update(heads=5), "divisible"),
    (lambda r: r.pop("canon"), "canon"),
    (lambda r: r.update(width=0), "width"),
])
def test_configurations_that_cannot_be_are_refused_by_name(change, word):
    raw = copy.deepcopy(TINY_P)
    change(raw)
    with pytest.raises(ConfigError, match=word):
        GufasunConfig.from_dict(raw)


def test_recipe_names_every_tensor_with_its_shape():
    c = GufasunConfig.from_dict(TINY_P)
    spec = detect_architecture(c.to_dict()).recipe(c, ())
    t = {n: tuple(d.shape) for n, d in expected_checkpoint_tensors(spec).items()}
    assert t["embed"] == (211, 72) and t["head"] == (211, 72) and t["final.norm"] == (72,)
    assert t["l0.mix.q"] == (96, 72) and t["l0.mix.k"] == (32, 72) and t["l0.mix.v"] == (64, 72)
    assert t["l0.mix.q.conv"] == (96, 3) and t["l0.mix.v.b"] == (64,) and t["l0.mix.k.norm"] == (16,)
    assert t["l0.mix.r1"] == (6,) and t["l0.mix.o"] == (72, 192) and t["l0.canon1"] == (72, 3)
    assert t["l1.mix.i"] == (3, 72) and t["l1.mix.f.b"] == (3,) and t["l1.mix.norm"] == (60,) and t["l1.mix.g"] == (60, 72)
    assert t["l1.mlp.up"] == (88, 72) and t["l1.mlp.down.b"] == (72,) and t["l1.mlp.act"] == (4,)
    # the layer that reads another one's keys and values has none of its own; the layer without a feed-forward no second norm
    assert not [n for n in t if n.startswith("l2.mix.k") or n.startswith("l2.mix.v")]
    assert "l2.mix.q.norm" in t and "l3.norm2" not in t and not [n for n in t if n.startswith("l3.mlp")]
    assert [e.cache_from for e in spec.schedule] == [None, None, 0, None]


def test_cache_needs_are_trees_and_a_reader_keeps_its_own_state_beside_the_pages_it_borrows():
    c = GufasunConfig.from_dict(TINY_P)
    spec = detect_architecture(c.to_dict()).recipe(c, ())
    needs = declared_cache_needs(spec)
    kv = needs[0]["inner"]["kv"]
    assert isinstance(kv, PagedNeed) and kv.window == 21 and [t.name for t in kv.page_tensors()] == ["k", "v"]
    assert needs[0]["inner"]["conv"] == StateNeed((2, 96 + 32 + 64), None) and needs[0]["input_conv"] == StateNeed((2, 72), None)
    assert set(needs[1]["inner"]) == {"S", "n", "m"} and needs[1]["inner"]["S"].shape == (3, 12, 20)
    assert needs[2] == {"inner": {"conv": StateNeed((2, 96), None)}, "input_conv": StateNeed((2, 72), None)}
    assert [p for p, _ in need_leaves(needs[2])] == [("inner", "conv"), ("input_conv",)]

    cache = CacheManager(needs, page_size=4, num_pages=8, max_slots=2, max_request_tokens=32,
                         readers={2: 0})
    assert len(cache.groups) == 1
    own, lent = cache.view(0), cache.view(2)
    assert isinstance(own["inner"]["kv"], PagedView) and own["inner"]["kv"].writes
    assert isinstance(lent["inner"]["kv"], PagedView) and not lent["inner"]["kv"].writes and lent["inner"]["kv"].window == 21
    assert isinstance(lent["inner"]["conv"], StateView) and isinstance(lent["input_conv"], StateView)
    assert isinstance(cache.view(1)["inner"]["m"], StateView)
    cache.admit("a")
    cache.append([("a", 30)])
    cache.trim_windows("a")
    assert cache.table_of("a").count(-1) == (30 - 21 + 1) // 4      # pages that the wider window has passed
    cache.release("a")
    cache.check()


def test_a_single_need_still_stands_alone():
    cache = CacheManager([StateNeed((3,), torch.float32), PagedNeed(2, 8), None], page_size=4, num_pages=4, max_slots=2,
                         max_request_tokens=16, readers={2: 1})
    assert isinstance(cache.view(0), StateView) and cache.view(1).writes and not cache.view(2).writes


def test_the_command_line_writes_a_random_model_folder_of_this_design(tmp_path, capsys):
    import json
    import os

    from safetensors.torch import load_file

    from arle_amd.cli import main

    config = tmp_path / "config.json"
    config.write_text(json.dumps(TINY_Q))
    out = str(tmp_path / "model")
    assert main(["random-weights", "--config", str(config), "--out", out, "--seed-weights", "3"]) == 0
    assert capsys.readouterr().out.strip() == out
    assert json.load(open(os.path.join(out, "config.json")))["architecture"] == "Gufasun"
    names = set(load_file(os.path.join(out, "model.safetensors")))
    assert {"embed", "head", "final.norm", "l0.mix.i.b", "l1.mix.r2", "l2.mix.k.conv", "l2.canon1"} <= names
    assert "l1.mix.q.conv" not in names       # that layer has no convolution on q, k and v
    # a folder of this design that is damaged ends like any other: one line, exit code 1
    bad = dict(TINY_Q, layers=[dict(TINY_Q["layers"][0], type="gru")])
    (tmp_path / "bad").mkdir()
    (tmp_path / "bad" / "config.json").write_text(json.dumps(bad))
    assert main(["--model-path", str(tmp_path / "bad"), "run", "--prompt-ids", "1,2"]) == 1
    assert "unknown layer type" in capsys.readouterr().err

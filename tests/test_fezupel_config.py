"""The Fezupel configuration on the CPU: what config.json gives, what it refuses, the order
of the layers' runs, the tensors a model declares, and a model folder written and read."""
import copy
import json
import os

import pytest
import torch

import fezupel_tiny as fz
import plain_fezupel
from zinfer_amd.config import (FezupelConfig, LayerNormSpec, MoeSpec, SandwichNormBlockSpec,
                               TiedKeyValueAttentionSpec, entry_for)
from zinfer_amd.errors import ConfigError
from zinfer_amd.models.build import declare_tensors


def test_registry_finds_the_family_by_its_one_name():
    assert entry_for(fz.FZ_A).config_type is FezupelConfig
    assert entry_for({"architecture": "Fezupel", "model_type": "qwen3"}).config_type is FezupelConfig


@pytest.mark.parametrize("name", sorted(fz.CONFIGS))
def test_sizes_and_constants_come_from_the_file(name):
    raw = fz.CONFIGS[name]
    cfg = fz.config_of(name)
    spec = cfg.model_spec()
    assert (spec.vocab_size, spec.hidden_size, spec.max_positions) == \
        (raw["vocab"], raw["width"], raw["max_positions"])
    assert spec.position_table_name == "pos" and not spec.tie_word_embeddings
    assert isinstance(spec.final_norm, LayerNormSpec) and spec.final_norm.eps == raw["norm"]["eps"]
    for L, block in zip(raw["layers"], spec.layers):
        assert isinstance(block, SandwichNormBlockSpec)
        m = block.mixer
        assert isinstance(m, TiedKeyValueAttentionSpec) and m.sink and m.output_gate
        assert (m.n_heads, m.n_kv_heads, m.head_dim, m.window, m.scale) == \
            (L["mixer"]["heads"], L["mixer"]["kv_heads"], L["mixer"]["dim"],
             L["mixer"]["mask"]["size"], L["mixer"]["scale"])
        if L["mlp"] is None:
            assert block.feed_forward is None and block.ff_norm is None
        else:
            f = block.feed_forward
            assert isinstance(f, MoeSpec) and f.router_bias
            assert (f.n_experts, f.top_k) == (L["mlp"]["router"]["experts"], L["mlp"]["router"]["top"])
            assert (f.expert.intermediate_size, f.expert.limit) == \
                (L["mlp"]["expert"]["ff"], L["mlp"]["expert"]["limit"])
            assert (f.expert.alpha, f.expert.shift) == (1.702, 1.0)
            if L["mlp"]["shared"] is None:
                assert f.shared is None
            else:
                assert (f.shared.intermediate_size, f.shared.limit) == \
                    (L["mlp"]["shared"]["ff"], L["mlp"]["shared"]["limit"])


def test_layer_order_follows_the_loop():
    assert fz.config_of("A").layer_order() == (0, 0, 0, 1)
    assert fz.config_of("B").layer_order() == (0, 1, 2)
    assert fz.config_of("C").layer_order() == (0, 1)
    assert fz.config_of("D").layer_order() == (0, 1, 2, 1, 2, 3)
    for name in fz.CONFIGS:
        assert list(fz.config_of(name).layer_order()) == plain_fezupel.layer_order(fz.CONFIGS[name])
        # every run has a cache of its own
        assert all(e.cache_of is None for e in fz.config_of(name).model_spec().schedule)


def test_declared_tensors_and_their_shapes():
    d = declare_tensors(fz.config_of("B").model_spec())
    assert d["embed"].shape == (300, 72) and d["pos"].shape == (256, 72) and d["head"].shape == (300, 72)
    assert d["final.norm"].shape == (72,) and d["final.norm.b"].shape == (72,)
    assert d["l0.mix.q"].shape == (48, 72) and d["l0.mix.k"].shape == (48, 72)
    assert d["l1.mix.q"].shape == (48, 72) and d["l1.mix.k"].shape == (16, 72)
    assert d["l1.mix.g"].shape == (48, 72) and d["l1.mix.o"].shape == (72, 48)
    assert "l0.mix.v" not in d
    assert not any(n.startswith("l1.mlp") or n.startswith("l1.norm2") for n in d)
    assert d["l2.mlp.router"].shape == (9, 72) and d["l2.mlp.router.b"].shape == (9,)
    assert d["l2.mlp.e8.gate"].shape == (16, 72) and d["l2.mlp.e8.down"].shape == (72, 16)
    assert d["l2.mlp.shared.up"].shape == (8, 72) and "l0.mlp.shared.up" not in d
    for k in ("norm1", "norm1b", "norm2", "norm2b"):
        assert d[f"l0.{k}"].shape == (72,) and d[f"l0.{k}.b"].shape == (72,)


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][0].update(type="recurrent"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=5), "vdim"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=99), "top"),
    (lambda c: c["layers"][0]["mlp"]["expert"].update(limit=0), "limit"),
    (lambda c: c.update(loop={"start": 1, "stop": 9, "times": 2}), "loop"),
    (lambda c: c.update(width="wide"), "width"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_what_the_formulas_do_not_cover_is_refused(change, text):
    raw = copy.deepcopy(fz.FZ_A)
    change(raw)
    with pytest.raises(ConfigError, match=text):
        FezupelConfig.from_dict(raw)


def test_model_folder_written_and_read(tmp_path):
    from zinfer_amd.config import load_config
    from zinfer_amd.weights import write_model_dir
    from zinfer_amd.weights.loader import load_tensors
    cfg = fz.config_of("A")
    path = write_model_dir(str(tmp_path / "m"), cfg, 3, torch.bfloat16)
    again = load_config(path)
    assert isinstance(again, FezupelConfig) and again.layers == cfg.layers and again.loop == cfg.loop
    tensors = load_tensors(path, declare_tensors(again.model_spec()))
    assert tensors["l1.mlp.e4.down"].dtype == torch.bfloat16
    assert float(tensors["l0.norm1b.b"].float().abs().max()) > 0.0


def test_plain_layer_pieces():
    """The oracle against itself where a piece has a closed form."""
    x = torch.tensor([[1.0, 2.0, 3.0, 6.0]])
    n = plain_fezupel.layer_norm(x, torch.ones(4), torch.zeros(4), 0.0)
    assert abs(float(n.mean())) < 1e-12 and abs(float((n * n).mean()) - 1.0) < 1e-12
    # one key, score 0: the silent term takes half of the weight
    q = torch.zeros((1, 4)); k = torch.tensor([[2.0, 4.0, 6.0, 8.0]])
    o = plain_fezupel.sink_window_attention(q, k, 1, 1, 4, 1.0, 3)
    assert torch.allclose(o, k.double() / 2)


def test_command_line_writes_and_inspects_a_model_folder(tmp_path, capsys):
    from zinfer_amd.cli import main
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(fz.FZ_B))
    out = str(tmp_path / "m")
    assert main(["random-model", str(cfg), out, "--seed", "4", "--dtype", "float32"]) == 0
    assert main(["inspect-config", out]) == 0
    text = capsys.readouterr().out
    assert "architecture: Fezupel" in text and "width: 72" in text and "model_type: fezupel" in text
    assert text.count("architecture:") == 1
    assert main(["inspect-weights", out]) == 0
    text = capsys.readouterr().out
    assert "tensor l0.mlp.router.b: dtype=F32 shape=[3] " in text

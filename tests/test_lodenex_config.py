"""The Lodenex configuration on the CPU: what config.json gives, what it refuses, the rules
for the rotations' frequencies against the plain implementation's, the cache each mixer asks
for, the tensors a model declares, and a model folder written and read."""
import copy
import json
import math
import os

import pytest
import torch

import lodenex_tiny as lx
import plain_lodenex as P
from zinfer_amd.config import (DenseMlpSpec, LatentAttentionSpec, LayerNormSpec, LodenexConfig,
                               MaskedGqaAttentionSpec, PostNormBlockSpec, entry_for)
from zinfer_amd.config import rotary
from zinfer_amd.errors import ConfigError
from zinfer_amd.models.build import declare_tensors
from zinfer_amd.parts.base import KVNeed


def test_registry_finds_the_family_by_its_one_name():
    assert entry_for(lx.LX_A).config_type is LodenexConfig
    assert entry_for({"architecture": "Lodenex", "model_type": "qwen3"}).config_type is LodenexConfig


@pytest.mark.parametrize("name", sorted(lx.CONFIGS))
def test_sizes_and_constants_come_from_the_file(name):
    raw = lx.CONFIGS[name]
    spec = lx.config_of(name).model_spec()
    assert (spec.vocab_size, spec.hidden_size) == (raw["vocab"], raw["width"])
    assert spec.embedding_multiplier == raw["embedding"]["scale"]
    assert spec.logit_softcap == raw["logit_softcap"] and spec.position_table_name is None
    assert isinstance(spec.final_norm, LayerNormSpec) and spec.final_norm.eps == raw["norm"]["eps"]
    assert not spec.final_norm.centred and spec.final_norm.bias_name is None
    assert [e.layer for e in spec.schedule] == list(range(len(raw["layers"])))
    for L, block in zip(raw["layers"], spec.layers):
        assert isinstance(block, PostNormBlockSpec)
        m, r = block.mixer, L["mixer"]
        if L["type"] == "attention":
            assert isinstance(m, MaskedGqaAttentionSpec) and m.sink and m.head_gate
            assert (m.n_heads, m.n_kv_heads, m.head_dim, m.value_dim, m.scale, m.softcap, m.chunk,
                    m.window, m.qk_norm_eps) == \
                (r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["scale"], r["softcap"],
                 r["mask"]["size"], None, raw["norm"]["eps"])
            assert m.rotary.dims == r["rot"]["dims"] and m.rotary.magnitude == 1.0
        else:
            assert isinstance(m, LatentAttentionSpec) and m.element_gate
            assert (m.n_heads, m.head_dim, m.rot_dim, m.value_dim, m.q_rank, m.kv_rank, m.scale,
                    m.window, m.chunk, m.norm_eps) == \
                (r["heads"], r["dim"], r["rot_dim"], r["vdim"], r["q_rank"], r["kv_rank"],
                 r["scale"], r["mask"]["size"], None, raw["norm"]["eps"])
            assert m.rotary.dims == r["rot_dim"]
        if L["mlp"] is None:
            assert block.feed_forward is None and block.ff_post_norm is None
        else:
            f = block.feed_forward
            assert isinstance(f, DenseMlpSpec) and f.activation == "gelu"
            assert f.intermediate_size == L["mlp"]["ff"]


def test_frequency_rules_against_the_plain_ones():
    """Both rules, written twice (here and in the plain implementation), on shapes that reach
    every branch: kept, slowed, blended; before, on and behind the ramp."""
    seen = set()
    for raw in lx.CONFIGS.values():
        for L in raw["layers"]:
            rot = L["mixer"]["rot"]
            spec = rotary.leading_rotary(rot["base"], rot["dims"], rot["scaling"])
            sc = rot["scaling"]
            if sc is None:
                want, mag = P.base_frequencies(rot["base"], rot["dims"]), 1.0
                seen.add("plain")
            elif "low" in sc:
                want, mag = P.wavelength_scaled_frequencies(rot["base"], rot["dims"], sc), 1.0
                plain = P.base_frequencies(rot["base"], rot["dims"])
                for f, p in zip(want.tolist(), plain.tolist()):
                    seen.add("kept" if f == p else "slowed" if abs(f - p / sc["factor"]) < 1e-15 * p
                             else "blended")
            else:
                want, mag = P.yarn_frequencies(rot["base"], rot["dims"], sc)
                plain = P.base_frequencies(rot["base"], rot["dims"])
                for f, p in zip(want.tolist(), plain.tolist()):
                    seen.add("fast" if f == p else "slow" if abs(f - p / sc["factor"]) < 1e-15 * p
                             else "ramp")
                assert mag == pytest.approx(0.1 * math.log(sc["factor"]) + 1.0, rel=1e-15)
            assert spec.magnitude == pytest.approx(mag, rel=1e-15)
            assert torch.allclose(torch.tensor(spec.frequencies, dtype=torch.float64), want,
                                  rtol=1e-14, atol=0)
    assert seen >= {"plain", "kept", "slowed", "blended", "fast", "slow", "ramp"}, seen


def test_frequency_rules_by_hand():
    f = rotary.plain_frequencies(100.0, 4)
    assert f == (1.0, pytest.approx(0.1))
    # wavelengths 2 pi and 20 pi against original 32: 32/4 = 8 > 2 pi keeps, 32/1 < 20 pi slows
    assert rotary.by_wavelength(f, 8.0, 1.0, 4.0, 32.0) == (1.0, pytest.approx(0.0125))
    # between: wavelength 20 pi, original 128: t = (128 / (20 pi) - 1) / 3
    t = (128.0 / (20.0 * math.pi) - 1.0) / 3.0
    got = rotary.by_wavelength(f, 8.0, 1.0, 4.0, 128.0)[1]
    assert got == pytest.approx((1 - t) * 0.1 / 8.0 + t * 0.1)
    fr, mag = rotary.by_turns((1.0, 0.5, 0.25, 0.125), 16.0, 8, 4.0, 64.0, 4.0, 1.0)
    first = max(math.floor(8 * math.log(64.0 / (2 * math.pi * 4.0)) / (2 * math.log(16.0))), 0)
    last = min(math.ceil(8 * math.log(64.0 / (2 * math.pi * 1.0)) / (2 * math.log(16.0))), 7)
    assert (first, last) == (1, 4)
    assert fr == pytest.approx((1.0, 0.5, 0.25 * (1 / 3 / 4 + 2 / 3), 0.125 * (2 / 3 / 4 + 1 / 3)))
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    with pytest.raises(ConfigError):
        rotary.leading_rotary(100.0, 6, {"factor": 2.0})
    with pytest.raises(ConfigError):
        rotary.plain_frequencies(100.0, 5)


def test_what_the_configuration_refuses():
    def broken(change):
        raw = copy.deepcopy(lx.LX_A)
        change(raw)
        with pytest.raises(ConfigError):
            LodenexConfig.from_dict(raw)
    broken(lambda r: r.pop("vocab"))
    broken(lambda r: r.update(width=0))
    broken(lambda r: r["norm"].update(eps=-1.0))
    broken(lambda r: r.update(layers=[]))
    broken(lambda r: r["layers"][0].update(type="recurrent"))
    broken(lambda r: r["layers"][0]["mixer"].update(kv_heads=3))
    broken(lambda r: r["layers"][0]["mixer"]["rot"].update(dims=14))     # more than a head
    broken(lambda r: r["layers"][0]["mixer"]["rot"].update(dims=5))
    broken(lambda r: r["layers"][0]["mixer"].update(softcap=0.0))
    broken(lambda r: r["layers"][0]["mixer"]["mask"].update(size=0))
    broken(lambda r: r["layers"][0]["mlp"].update(kind="moe"))
    broken(lambda r: r["layers"][1]["mixer"]["rot"].update(dims=2))      # not the rotated part
    broken(lambda r: r["layers"][1]["mixer"].pop("kv_rank"))
    broken(lambda r: r.update(logit_softcap=-3.0))
    broken(lambda r: r["layers"][0]["mixer"]["rot"].update(scaling={"factor": 2.0, "bogus": 1}))


def test_cache_needs_and_declared_tensors():
    from zinfer_amd.models.decoder import DecoderModel
    from zinfer_amd.parts import BuildContext
    cfg = lx.config_of("A")
    model = DecoderModel(cfg.model_spec(), BuildContext(torch.float32, torch.device("meta")))
    assert model.cache_needs() == [KVNeed(2, 12, None, value_dim=20, chunk=7),
                                   KVNeed(1, 28, 5, value_dim=0),
                                   KVNeed(1, 16, None, value_dim=8, chunk=11)]
    d = {k: v.shape for k, v in declare_tensors(cfg.model_spec()).items()}
    assert d["embed"] == (211, 48) and d["head"] == (211, 48) and d["final.norm"] == (48,)
    assert d["l0.mix.q"] == (48, 48) and d["l0.mix.k"] == (24, 48) and d["l0.mix.v"] == (40, 48)
    assert d["l0.mix.q.norm"] == (48,) and d["l0.mix.k.norm"] == (24,)
    assert d["l0.mix.sink"] == (4,) and d["l0.mix.g"] == (4, 48) and d["l0.mix.o"] == (48, 80)
    assert d["l0.mlp.up"] == (40, 48) and d["l0.mlp.down"] == (48, 40)
    assert d["l1.mix.dq"] == (20, 48) and d["l1.mix.dq.norm"] == (20,)
    assert d["l1.mix.uq"] == (36, 20) and d["l1.mix.dkv"] == (28, 48)
    assert d["l1.mix.dkv.norm"] == (24,) and d["l1.mix.uk"] == (24, 24)
    assert d["l1.mix.uv"] == (30, 24) and d["l1.mix.g"] == (30, 48) and d["l1.mix.o"] == (48, 30)
    assert "l1.mlp.up" not in d and "l1.norm2" not in d and d["l1.norm1"] == (48,)
    assert len(d) == 3 + 12 + 10 + 12


def test_a_folder_written_and_read(tmp_path):
    from zinfer_amd.config import load_config
    from zinfer_amd.weights.loader import load_tensors
    from zinfer_amd.weights.safetensors_io import write_safetensors
    path = str(tmp_path)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(lx.LX_C, f)
    w = lx.weights_of("C", dtype=torch.bfloat16)
    write_safetensors(os.path.join(path, "model.safetensors"), w)
    cfg = load_config(path)
    assert isinstance(cfg, LodenexConfig) and cfg.to_dict() == lx.LX_C
    got = load_tensors(path, declare_tensors(cfg.model_spec()))
    assert set(got) == set(w) and all(torch.equal(got[k], w[k]) for k in w)


def test_the_plain_masks_and_the_sink():
    """The oracle's own pieces, by hand: who sees whom, and what the sink does to the weights."""
    c = P.chunk_mask(7, 3)
    assert c[2].tolist() == [True, True, True, False, False, False, False]
    assert c[3].tolist() == [False, False, False, True, False, False, False]
    assert c[6].tolist() == [False] * 6 + [True]
    wm = P.window_mask(6, 2)
    assert wm[0].tolist() == [True] + [False] * 5 and wm[4].tolist() == [False] * 3 + [True, True, False]
    s = torch.zeros((1, 2, 2), dtype=torch.float64)
    v = torch.tensor([[[1.0], [3.0]]], dtype=torch.float64)
    mask = P.window_mask(2, 2)
    out = P.masked_softmax_values(s, mask, v, torch.tensor([0.0]))
    assert out[0, 0, 0] == pytest.approx(0.5) and out[0, 1, 0] == pytest.approx(4.0 / 3.0)
    out = P.masked_softmax_values(s, mask, v, torch.tensor([math.log(2.0)]))
    assert out[0, 0, 0] == pytest.approx(1.0 / 3.0) and out[0, 1, 0] == pytest.approx(1.0)
    assert P.tanh_cap(torch.tensor(1000.0), 5.0) == pytest.approx(5.0)
    assert float(P.gelu_erf(torch.tensor(1.0, dtype=torch.float64))) == pytest.approx(0.8413447460685429)


def test_command_line_writes_and_inspects_a_model_folder(tmp_path, capsys):
    from zinfer_amd.cli import main
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(lx.LX_B))
    out = str(tmp_path / "m")
    assert main(["random-model", str(cfg), out, "--seed", "4", "--dtype", "float32"]) == 0
    assert main(["inspect-config", out]) == 0
    text = capsys.readouterr().out
    assert "architecture: Lodenex" in text and "width: 72" in text and "model_type: lodenex" in text
    assert text.count("architecture:") == 1
    assert main(["inspect-weights", out]) == 0
    text = capsys.readouterr().out
    assert "tensor l0.mix.dkv.norm: dtype=F32 shape=[32] " in text
    assert "tensor l0.mix.uk: dtype=F32 shape=[32, 32] " in text and "tensor_count: 50" in text

"""CPU tests of the layered-model family's host side: configuration parsing, tensor tables, checkpoint files, the registry, and
the float64 oracle's own consistency (a prompt fed whole, in portions, and token by token gives the same logits)."""
import json
import os
import struct

import numpy as np
import pytest

import lm_oracle
import lm_testlib as tl
from zig_gpt2_amd import lm, models, weights_io


def _cfg():
    return tl.config([tl.hgrn2_layer(mlp=tl.dense_mlp()), tl.latent_layer(mlp=tl.moe_mlp()), tl.latent_layer(rot_dim=12, rot_dims=8, scaling=None),
                      tl.hgrn2_layer(heads=1, dim=20, vdim=8, mlp=tl.moe_mlp(top=1))], loop={"start": 1, "stop": 3, "times": 3})


def test_config_round_trip_and_passes():
    cfg = _cfg()
    c = lm.LMConfig.from_json(cfg)
    assert c.to_json() == cfg
    assert c.passes() == lm_oracle.layer_runs(cfg) == [0, 1, 2, 1, 2, 1, 2, 3]
    assert lm.LMConfig.from_json(tl.config([tl.hgrn2_layer()])).passes() == [0]
    l1 = c.layers[1].to_c()
    assert (l1.mixer, l1.heads, l1.kv_rank, l1.rot_scaled, l1.ff, l1.experts, l1.top) == (2, 3, 40, 1, 2, 5, 2)
    l2 = c.layers[2].to_c()
    assert (l2.rot_dim, l2.rot_dims, l2.rot_scaled, l2.ff) == (12, 8, 0, 0)


def test_tensor_table_matches_oracle_needs():
    cfg = _cfg()
    w = tl.weights(cfg, seed=3)
    shapes = lm.LMConfig.from_json(cfg).tensor_shapes()
    assert set(w) == set(shapes)
    assert "l2.norm2" not in shapes and "l0.norm2" in shapes  # no feed-forward: no norms around it
    assert shapes["l1.mix.uq"] == (3 * (16 + 8), 48) and shapes["l1.mix.dkv"] == (40 + 8, 48)
    # the oracle runs on exactly these tensors
    lg, _ = lm_oracle.Model(cfg, w).forward(tl.tokens(0, 5, cfg["vocab"]))
    assert lg.shape == (5, cfg["vocab"]) and np.isfinite(lg).all()


def test_unknown_names_are_refused():
    bad = _cfg()
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        lm.LMConfig.from_json(bad)
    bad = _cfg()
    bad["layers"][0]["mlp"]["kind"] = "glu"
    with pytest.raises(ValueError):
        lm.LMConfig.from_json(bad)


def test_safetensors_round_trip(tmp_path):
    cfg = _cfg()
    w = tl.weights(cfg, seed=1)
    w["table"] = np.arange(12, dtype=np.int32).reshape(3, 4)
    p = str(tmp_path / "model.safetensors")
    weights_io.write_safetensors(p, w)
    raw = weights_io.read_safetensors(p)
    assert raw["embed"][0] == "BF16" and raw["embed"][1].dtype == np.uint16 and raw["table"][0] == "I32"
    back = weights_io.load_safetensors_f32(p)
    assert set(back) == set(w)
    for k in w:
        assert back[k].shape == w[k].shape and np.array_equal(back[k], w[k]), k  # bf16-representable values survive exactly
    weights_io.write_safetensors(p, {"a": np.float32([[1.00390625, 3.0]])}, bf16=False)
    assert weights_io.read_safetensors(p)["a"][0] == "F32" and weights_io.load_safetensors_f32(p)["a"][0, 0] == np.float32(1.00390625)


def test_safetensors_rejects_broken_files(tmp_path):
    p = str(tmp_path / "x.safetensors")
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 1 << 40))
    with pytest.raises(ValueError):
        weights_io.read_safetensors(p)
    head = json.dumps({"a": {"dtype": "BF16", "shape": [4], "data_offsets": [0, 8]}}).encode()
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", len(head)) + head + b"\0" * 6)  # two bytes short
    with pytest.raises(ValueError):
        weights_io.read_safetensors(p)


def test_registry_by_config_json(tmp_path):
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(_cfg()))
    assert models.architecture_of(str(d)) == "Tokosun"
    (d / "config.json").write_text(json.dumps({"architecture": "nope"}))
    with pytest.raises(ValueError):
        models.architecture_of(str(d))
    raw = tmp_path / "raw"
    raw.mkdir()
    (raw / "model-wte").write_bytes(b"")
    assert models.architecture_of(str(raw)) == "gpt2"
    assert set(models.ARCHITECTURES) >= {"Tokosun", "gpt2"}


def test_oracle_portions_agree():
    cfg = _cfg()
    m = lm_oracle.Model(cfg, tl.weights(cfg, seed=2))
    toks = tl.tokens(4, 19, cfg["vocab"])
    whole, _ = m.forward(toks)
    st, rows = None, []
    for lo, hi in [(0, 1), (1, 3), (3, 10), (10, 12), (12, 19)]:
        lg, st = m.forward(toks[lo:hi], st)
        rows.append(lg)
    assert np.abs(np.concatenate(rows) - whole).max() < 1e-9
    st, rows = None, []
    for t in toks:
        lg, st = m.forward([t], st)
        rows.append(lg)
    assert np.abs(np.concatenate(rows) - whole).max() < 1e-9


def test_oracle_rotary_blend_limits():
    # no scaling: plain frequencies base^(-2i/dims), amplitude one
    cos, sin = lm_oracle.rotary_tables({"dims": 8, "base": 100.0}, [0, 3])
    assert np.allclose(cos[0], 1.0) and np.allclose(sin[0], 0.0)
    assert np.allclose(cos[1], np.cos(3 * 100.0 ** (-np.arange(4) / 4.0)), atol=1e-6)
    # scaled: the fastest pair keeps its frequency, the slowest is divided by the factor, both carry the amplitude
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 16, "fast": 8.0, "slow": 0.5}}
    cos, sin = lm_oracle.rotary_tables(rot, [1])
    amp = 0.1 * np.log(4.0) + 1.0
    assert np.isclose(cos[0, 0], np.cos(1.0) * amp, atol=1e-6) and np.isclose(sin[0, 3], np.sin(100.0 ** (-0.75) / 4.0) * amp, atol=1e-6)

"""The Gupizen design without a GPU: configuration and tensor table of zig_gpt2_amd/lm.py, the registry, and the float64 oracle's
own properties (tests/gupizen_oracle.py) — portions against whole prompts, the window's edge, the sink, the bands of the
rotary frequencies, the router."""
import json
import os

import numpy as np
import pytest

import gupizen_oracle as go
import gupizen_testlib as gl
from zig_gpt2_amd import lm, models, weights_io


def full_cfg(**kw):
    return gl.config([gl.parallel_layer(mlp=gl.moe_mlp()), gl.delta_layer(mlp=gl.moe_mlp(experts=7, top=3)), gl.parallel_layer(heads=2, kv_heads=2, window=0, mlp=None),
                      gl.delta_layer(heads=3, kv_heads=3, dim=10, vdim=6, conv=2, mlp=gl.moe_mlp(top=1))], **kw)


def test_config_round_trip_and_tensor_table(tmp_path):
    cfg = full_cfg(loop={"start": 1, "stop": 3, "times": 3})
    c = lm.LMConfig.from_json(cfg)
    assert c.architecture == "Gupizen" and c.tied_head and c.canon_taps == 3 and abs(c.embed_scale - 0.7) < 1e-12
    assert c.passes() == [0, 1, 2, 1, 2, 1, 2, 3]
    assert lm.LMConfig.from_json(c.to_json()) == c
    t = c.tensor_shapes()
    assert "head" not in t and "l0.shift" not in t and t["l0.canon1"] == (48, 3) and "l2.canon2" not in t and "l2.norm2" not in t
    assert t["l0.mix.left.k"] == (2 * 12, 48) and t["l0.mix.right.ra"] == (2, 10, 10) and t["l1.mix.a2"] == (4 * 8, 6)
    assert t["l1.mlp.router.b"] == (7,) and "l1.mlp.e0.gate" not in t and "l1.mlp.correction" not in t
    l0 = c.layers[0].to_c()
    assert l0.window == 7 and l0.kv_heads == 2 and l0.rot_scaled == 2 and l0.rot_fast == 8.0 and l0.rot_slow == 1.0
    # the inner sizes of the two-step projections are not in a checkpoint's configuration: they come from the tensor shapes
    w = gl.weights(cfg, seed=1)
    for e in cfg["layers"]:
        e["mixer"].pop("decay_rank", None)
        e["mixer"].pop("gate_rank", None)
    with pytest.raises(KeyError):
        lm.LMConfig.from_json(cfg)
    d = tmp_path / "ckpt"
    os.makedirs(d)
    json.dump(cfg, open(d / "config.json", "w"))
    weights_io.write_safetensors(str(d / "model.safetensors"), w)
    c2 = lm.LMConfig.from_dir(str(d))
    assert c2.layers[1].decay_rank == 6 and c2.layers[1].gate_rank == 5 and c2 == c
    assert models.architecture_of(str(d)) == "Gupizen"


def test_oracle_portions_equal_whole_prompt():
    cfg = full_cfg(loop={"start": 0, "stop": 2, "times": 2})
    m = go.Model(cfg, gl.weights(cfg, seed=2))
    toks = gl.tokens(1, 40, cfg["vocab"])
    ref, _, layers = m.forward(toks, want_layers=True)
    assert layers.shape == (6, 40, 48)
    for cuts in ([2, 4, 5, 19, 33], list(range(1, 40))):
        st, rows, lo = None, [], 0
        for hi in cuts + [40]:
            out, st = m.forward(toks[lo:hi], st)
            rows.append(out)
            lo = hi
        assert np.abs(np.concatenate(rows) - ref).max() < 1e-9 * np.abs(ref).max()


def test_oracle_window_sink_and_mixed_heads():
    m = {"heads": 2, "kv_heads": 1, "scale": 1.0, "mask": {"size": 3}}
    q = np.zeros((5, 2, 4))
    k = np.zeros((5, 1, 4))
    ident = np.eye(2)
    a = go.window_attention_weights(q, k, m, np.array([-np.inf, 0.0]), ident, np.arange(5), np.arange(5))
    assert np.allclose(a[0, 4], [0, 0, 1 / 3, 1 / 3, 1 / 3]) and np.allclose(a[0, 1], [0.5, 0.5, 0, 0, 0])  # itself and two before
    assert np.allclose(a[1, 4], [0, 0, 0.25, 0.25, 0.25])  # exp(0) of the sink counts once, and has no value
    mixed = go.window_attention_weights(q, k, m, np.array([-np.inf, 0.0]), np.array([[1.0, 2.0], [0.0, -1.0]]), np.arange(5), np.arange(5))
    assert np.allclose(mixed[0, 4], a[0, 4] + 2 * a[1, 4]) and np.allclose(mixed[1, 4], -a[1, 4])


def test_oracle_frequency_bands():
    rot = {"base": 100.0, "dims": 8, "scaling": dict(gl.BANDS)}
    plain = np.array([100.0 ** (-2.0 * i / 8) for i in range(4)])
    f = go.band_scaled_frequencies(rot)
    wave = 2 * np.pi / plain
    assert wave[0] < 64 / 8 and wave[-1] > 64 / 1 and any(64 / 8 <= x <= 64 / 1 for x in wave), "the construction misses a band"
    assert f[0] == plain[0] and np.isclose(f[-1], plain[-1] / 4.0)
    mid = [i for i, x in enumerate(wave) if 64 / 8 <= x <= 64 / 1]
    assert all(plain[i] / 4.0 < f[i] < plain[i] for i in mid)


def test_oracle_router_and_recurrences():
    w = {"r.router": np.array([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]]), "r.router.b": np.array([0.0, 0.0, -10.0])}
    pick, wt = go.route_top_logits(np.array([[2.0, 1.0]]), w, "r.", 2)
    assert list(pick[0]) == [0, 1] and np.allclose(wt[0], np.exp([2.0, 1.0]) / np.exp([2.0, 1.0]).sum())
    # delta rule: writing (k, v) with beta = 1 into an empty state and reading with q = k returns v
    S, o = go.delta_step(np.zeros((3, 2)), np.array([0.0, 1.0, 0.0]), np.array([0.0, 1.0, 0.0]), np.array([5.0, 7.0]), 1.0, np.ones(3))
    assert np.allclose(o, [5.0, 7.0])
    S, o = go.delta_step(S, np.array([0.0, 1.0, 0.0]), np.array([0.0, 1.0, 0.0]), np.array([1.0, 1.0]), 1.0, np.array([1.0, 0.5, 1.0]))
    assert np.allclose(o, [1.0, 1.0])  # the decayed row is overwritten: the read-out sees the current token's write
    c, tail = go.causal_conv(np.arange(8.0).reshape(4, 2), np.array([[1.0, 10.0, 100.0]] * 2), None)
    assert np.allclose(c[:, 0], [0, 200, 420, 642]) and np.allclose(tail, [[4, 5], [6, 7]])

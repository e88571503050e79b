"""The Gupizen design on the layered-model tier (zig_gpt2_amd/lm.py) against the float64 oracle of tests/gupizen_oracle.py: every
mechanism alone, whole prompts against portions and token-by-token decoding, ragged batches, slots and pages that go round
(also pages a window has left behind), keys at the window's edge and sinks made to stand out, slow forgetting in both
recurrences, other sizes, and generation through the library's entry points, the scheduler, the host program and the trace
replay."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import gupizen_oracle as go
import gupizen_testlib as gl
import lm_testlib as tl
from zig_gpt2_amd import lm, models, weights_io

pytestmark = pytest.mark.gpu


def make(cfg, w, dtype="float32", **kw):
    kw.setdefault("max_tokens", 512)
    kw.setdefault("max_seqs", 4)
    m = lm.LayeredLM(lm.LMConfig.from_json(cfg), dtype=dtype, **kw)
    m.load_weights(w)
    return m


def run_whole(m, toks, want=None, trace=False):
    s = m.open()
    out = m.step([(s, toks, list(range(len(toks))) if want is None else want)], trace=trace)
    m.close_seq(s)
    return out


def run_cut(m, toks, cuts):
    """Feed toks in portions that end at `cuts`; all logits."""
    s = m.open()
    rows, lo = [], 0
    for hi in list(cuts) + [len(toks)]:
        if hi > lo:
            rows.append(m.step([(s, toks[lo:hi], list(range(hi - lo)))]))
        lo = hi
    m.close_seq(s)
    return np.concatenate(rows)


SINGLE = {
    "parallel": [gl.parallel_layer()],  # grouped keys, part of the head rotated, all three frequency bands, a window
    "parallel_plain": [gl.parallel_layer(heads=3, kv_heads=3, dim=8, vdim=12, window=0, rot_dims=8, scaling=None, blocks=1, conv=1)],
    "parallel_one_head": [gl.parallel_layer(heads=1, kv_heads=1, dim=6, vdim=4, window=70, rot_dims=2, width=7, blocks=7, conv=5)],  # a window beyond one key tile
    "delta": [gl.delta_layer()],
    "delta_own_keys": [gl.delta_layer(heads=3, kv_heads=3, dim=20, vdim=6, conv=1, decay_rank=1, gate_rank=9)],
    "delta_wide": [gl.delta_layer(heads=1, kv_heads=1, dim=72, vdim=40, conv=2)],  # more rows than a thread's share of one pass, columns beyond a power of two
    "moe": [gl.delta_layer(mlp=gl.moe_mlp())],
    "moe_top1": [gl.parallel_layer(mlp=gl.moe_mlp(ff=20, experts=3, top=1))],
    "moe_all": [gl.delta_layer(mlp=gl.moe_mlp(ff=8, experts=4, top=4))],
    "moe_many": [gl.delta_layer(mlp=gl.moe_mlp(ff=8, experts=70, top=3))],  # more experts than a wave has lanes
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_alone(name, dtype):
    cfg = gl.config(SINGLE[name], taps=2 if "plain" in name else 1 if "own_keys" in name else 3)
    w = gl.weights(cfg, seed=sum(map(ord, name)))
    toks = gl.tokens(1, 83 if "one_head" in name else 37, cfg["vocab"])
    ref, _, ref_tr = go.Model(cfg, w).forward(toks, want_layers=True)
    m = make(cfg, w, dtype)
    got, tr = run_whole(m, toks, trace=True)
    tl.assert_close(tr, ref_tr, dtype, "residual stream")
    tl.assert_close(got, ref, dtype, "logits")
    # the same prompt token by token: the decode kernels, state carried by the slot
    step = run_cut(m, toks, range(1, len(toks)))
    tl.assert_close(step, ref, dtype, "decoded")
    m.close()


def full_cfg(**kw):
    return gl.config([gl.parallel_layer(mlp=gl.moe_mlp()), gl.delta_layer(mlp=gl.moe_mlp(experts=7, top=3)),
                      gl.parallel_layer(heads=2, kv_heads=1, dim=10, vdim=14, window=19, rot_dims=10, width=24, blocks=3, conv=2, mlp=None),
                      gl.delta_layer(heads=3, kv_heads=1, dim=10, vdim=6, conv=2, mlp=gl.moe_mlp(top=1))], **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_several_sizes(dtype):
    cfg = full_cfg(loop={"start": 1, "stop": 3, "times": 2})
    w = gl.weights(cfg, seed=5)
    toks = gl.tokens(2, 90, cfg["vocab"])
    ref, _ = go.Model(cfg, w).forward(toks)
    m = make(cfg, w, dtype, page_tokens=8)
    tl.assert_close(run_whole(m, toks), ref, dtype)
    for cuts in ([2, 4, 7, 15, 16, 24, 25, 57, 88], [1, 2, 3, 40, 41, 43], list(range(9, 90, 9)), [64]):
        tl.assert_close(run_cut(m, toks, cuts), ref, dtype, cuts)
    # portions longer than one pass of the library are cut inside the step
    m2 = make(cfg, w, dtype, max_step_tokens=16, page_tokens=8)
    tl.assert_close(run_whole(m2, toks), ref, dtype)
    tl.assert_close(run_cut(m2, toks, [33, 35]), ref, dtype)
    m.close()
    m2.close()


def test_loop_variants_and_no_loop():
    """The embedding output is added in front of every repetition but the first: the oracle without it must differ."""
    for loop in (None, {"start": 0, "stop": 4, "times": 3}, {"start": 2, "stop": 3, "times": 2}, {"start": 0, "stop": 1, "times": 1},
                 {"start": 1, "stop": 4, "times": 2}):
        cfg = full_cfg(loop=loop, taps=4)
        w = gl.weights(cfg, seed=6)
        toks = gl.tokens(3, 21, cfg["vocab"])
        ref, _, ref_tr = go.Model(cfg, w).forward(toks, want_layers=True)
        m = make(cfg, w)
        got, tr = run_whole(m, toks, trace=True)
        assert tr.shape == ref_tr.shape
        tl.assert_close(tr, ref_tr, "float32", loop)
        tl.assert_close(got, ref, "float32", loop)
        tl.assert_close(run_cut(m, toks, [5, 6, 8]), ref, "float32", loop)
        m.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_batch(dtype):
    cfg = full_cfg(loop={"start": 0, "stop": 2, "times": 2})
    w = gl.weights(cfg, seed=7)
    oracle = go.Model(cfg, w)
    lens = [41, 3, 17, 1]
    prompts = [gl.tokens(10 + i, n, cfg["vocab"]) for i, n in enumerate(lens)]
    refs = [oracle.forward(p)[0] for p in prompts]
    m = make(cfg, w, dtype, page_tokens=4)
    seqs = [m.open() for _ in prompts]
    first = [30, 2, 9, 1]
    got = m.step([(s, p[:k], list(range(k))) for s, p, k in zip(seqs, prompts, first)])
    off = 0
    for r, k in zip(refs, first):
        tl.assert_close(got[off:off + k], r[:k], dtype)
        off += k
    entries = [(s, p[k:], list(range(len(p) - k))) for s, p, k in zip(seqs, prompts, first) if len(p) > k]
    got = m.step(entries)
    off = 0
    for r, p, k in zip(refs, prompts, first):
        if len(p) > k:
            tl.assert_close(got[off:off + len(p) - k], r[k:], dtype)
            off += len(p) - k
    # lock-step decoding of three sequences at different positions against each alone
    more = [gl.tokens(20 + i, 6, cfg["vocab"]) for i in range(3)]
    alone = [oracle.forward(np.concatenate([prompts[i], more[i]]))[0][len(prompts[i]):] for i in range(3)]
    rows = [m.step([(seqs[i], [more[i][t]], [0]) for i in range(3)]) for t in range(6)]
    for i in range(3):
        tl.assert_close(np.stack([r[i] for r in rows]), alone[i], dtype, i)
    m.close()


def test_slots_and_pages_are_reused():
    """Two slots and a cache of 64 tokens; every window is at most 19 tokens, so a sequence gives pages back while it grows."""
    cfg = full_cfg()
    w = gl.weights(cfg, seed=8)
    oracle = go.Model(cfg, w)
    m = make(cfg, w, max_tokens=64, max_seqs=2, page_tokens=4)
    total = m.free_tokens()
    a, b = gl.tokens(30, 33, cfg["vocab"]), gl.tokens(31, 26, cfg["vocab"])
    ra, rb = oracle.forward(a)[0], oracle.forward(b)[0]
    for rnd in range(3):
        sa, sb = m.open(), m.open()
        with pytest.raises(Exception):
            m.open()  # both slots taken
        got = m.step([(sa, a[:20], [19]), (sb, b[:5], [4])])
        tl.assert_close(got[0], ra[19], "float32")
        tl.assert_close(got[1], rb[4], "float32")
        m.close_seq(sb)  # its pages go to the other sequence, its slot to a new one
        got = m.step([(sa, a[20:], [12])])
        tl.assert_close(got[0], ra[32], "float32", rnd)
        assert total - m.free_tokens() <= 19 + 2 * 4  # the pages behind the longest window are back in the pool
        sb = m.open()
        got = m.step([(sb, b, list(range(len(b))))])
        tl.assert_close(got, rb, "float32", rnd)  # nothing of the slot's former sequence is left
        with pytest.raises(Exception):
            m.step([(sa, np.concatenate([a, a, a]), [])])  # more tokens than the cache has pages for
        assert m.seq_len(sa) == 33 and m.seq_len(sb) == 26
        m.close_seq(sa)
        m.close_seq(sb)
        assert m.free_tokens() == total
    # a sequence far longer than the cache: the window's pages go round
    long = gl.tokens(32, 300, cfg["vocab"])
    rl = oracle.forward(long)[0]
    s = m.open()
    rows = [m.step([(s, long[i:i + 10], list(range(10)))]) for i in range(0, 300, 10)]
    tl.assert_close(np.concatenate(rows), rl, "float32")
    m.close_seq(s)
    assert m.free_tokens() == total
    m.close()


def test_general_window_kernel(monkeypatch):
    """The one-workgroup-per-row form of the windowed attention (what a step takes when the split form's workspace would not
    fit), on prompts, portions and decoded tokens, windows of several key tiles included."""
    monkeypatch.setenv("ZGPT2_LM_WINDOW_GENERAL", "1")
    cfg = gl.config([gl.parallel_layer(window=0), gl.parallel_layer(heads=2, kv_heads=1, dim=70, vdim=6, window=90, rot_dims=30)])
    w = gl.weights(cfg, seed=21)
    toks = gl.tokens(22, 200, cfg["vocab"])
    ref = go.Model(cfg, w).forward(toks)[0]
    for dtype in ("float32", "bfloat16"):
        m = make(cfg, w, dtype)
        tl.assert_close(run_whole(m, toks), ref, dtype)
        tl.assert_close(run_cut(m, toks, [3, 64, 65, 130] + list(range(180, 200))), ref, dtype)
        m.close()


@pytest.mark.parametrize("hook", ["ZGPT2_LM_WINDOW_NO_TILES", "ZGPT2_LM_WINDOW_TILES"])
def test_both_score_kernels_on_all_steps(monkeypatch, hook):
    """Prompt portions take their scores from matrix-core tiles of 32 rows x 32 keys, steps of few rows from the wave-per-key
    kernel; the hooks send every step through one of them (ragged row blocks, windows that start inside a tile, two entries)."""
    monkeypatch.setenv(hook, "1")
    cfg = gl.config([gl.parallel_layer(heads=6, kv_heads=2, dim=18, vdim=4, window=41, rot_dims=6), gl.parallel_layer(heads=1, kv_heads=1, dim=5, vdim=2, window=0, rot_dims=4),
                     gl.parallel_layer(heads=18, kv_heads=6, dim=4, vdim=34, window=9, rot_dims=2)])  # more heads than the tiled value product takes
    w = gl.weights(cfg, seed=23)
    a, b = gl.tokens(24, 150, cfg["vocab"]), gl.tokens(25, 47, cfg["vocab"])
    oracle = go.Model(cfg, w)
    ra, rb = oracle.forward(a)[0], oracle.forward(b)[0]
    m = make(cfg, w)
    tl.assert_close(run_whole(m, a), ra, "float32")
    tl.assert_close(run_cut(m, a, [3, 35, 36, 100] + list(range(140, 150))), ra, "float32")
    sa, sb = m.open(), m.open()
    got = m.step([(sa, a[:70], list(range(70))), (sb, b, list(range(47)))])
    tl.assert_close(got[:70], ra[:70], "float32")
    tl.assert_close(got[70:], rb, "float32")
    m.close()


def _edge_model(window, n, seed):
    """One parallel layer whose attention is sharp (large score factor, no rotary on the scores' channels beyond two): most
    queries put nearly all their weight on one key.  Returns (cfg, weights, oracle, distance of the heaviest key per head and query)."""
    lay = gl.parallel_layer(heads=2, kv_heads=1, dim=16, vdim=8, window=window, scale=8.0, rot_dims=2, scaling=None)
    cfg = gl.config([lay], width=32)
    w = gl.weights(cfg, seed=seed, sink_mean=-8.0)
    w["l0.mix.left.talk"] = np.eye(2, dtype=np.float32)
    toks = gl.tokens(seed, n, cfg["vocab"])
    oracle = go.Model(cfg, w)
    x = oracle.w["embed"][toks] * 0.7
    h = go.norm_around_zero(x, oracle.w["l0.norm1"], oracle.eps)
    h = h + go.causal_conv(h, oracle.w["l0.canon1"], None)[0]
    m = lay["mixer"]["left"]
    q = (h @ oracle.w["l0.mix.left.q"].T).reshape(n, 2, 16)
    k = (h @ oracle.w["l0.mix.left.k"].T).reshape(n, 1, 16)
    ang = go.angles(np.arange(n), go.band_scaled_frequencies(m["rot"]))
    att = go.window_attention_weights(go.turn_pairs(q, ang, 2), go.turn_pairs(k, ang, 2), m, oracle.w["l0.mix.left.sink"], np.eye(2), np.arange(n),
                                      np.arange(n))
    return cfg, w, toks, oracle, att


def test_keys_at_the_windows_edge_stand_out():
    """A sharp softmax: a key that is one token too many or too few at the window's far edge, or read from a wrong page,
    changes a row by its whole value.  The same prompt with a window one token longer or shorter must differ clearly."""
    window, n = 23, 150
    cfg, w, toks, oracle, att = _edge_model(window, n, 9)
    top, far = att.max(axis=-1), np.arange(n)[None, :] - att.argmax(axis=-1)
    assert ((top > 0.8) & (far == window - 1)).sum() >= 3, "the construction puts no heavy key on the window's edge"
    ref = oracle.forward(toks)[0]
    for other in (window - 1, window + 1):
        cfg2 = json.loads(json.dumps(cfg))
        cfg2["layers"][0]["mixer"]["left"]["mask"]["size"] = other
        assert tl.rel_err(go.Model(cfg2, w).forward(toks)[0], ref) > 1e-2
    m = make(cfg, w, page_tokens=8)
    assert tl.rel_err(run_whole(m, toks), ref) < 2e-4
    assert tl.rel_err(run_cut(m, toks, [7, 8, 9, 22, 23, 24, 46, 100]), ref) < 2e-4
    assert tl.rel_err(run_cut(m, toks, range(60, n)), ref) < 2e-4  # decoded one by one, the window sliding over pages
    m.close()


def test_sink_takes_its_share():
    """Large sinks: most of a head's weight goes to the sink, which has no value — leaving it out would multiply the left
    branch's output severalfold."""
    cfg, w, toks, oracle, _ = _edge_model(12, 60, 10)
    w["l0.mix.left.sink"] = np.array([6.0, 9.0], np.float32)
    ref = go.Model(cfg, w).forward(toks)[0]
    w2 = dict(w)
    w2["l0.mix.left.sink"] = np.array([-30.0, -30.0], np.float32)
    assert tl.rel_err(go.Model(cfg, w2).forward(toks)[0], ref) > 1e-2, "the construction gives the sink no weight"
    m = make(cfg, w)
    tl.assert_close(run_whole(m, toks), ref, "float32")
    tl.assert_close(run_cut(m, toks, range(40, 60)), ref, "float32")
    m.close()


@pytest.mark.parametrize("kind", ["parallel", "delta"])
def test_recurrences_remember_far_tokens(kind):
    """Decays close to one: the recurrent state forgets slowly, so the first tokens still weigh in hundreds of tokens later
    (far beyond the window) — a state that is lost or reset between portions shows."""
    lay = gl.parallel_layer(window=5) if kind == "parallel" else gl.delta_layer(dim=16)
    cfg = gl.config([lay], width=32)
    w = gl.weights(cfg, seed=11, lam_mean=-7.0, a_log_mean=-6.0)
    n = 260
    toks = gl.tokens(41, n, cfg["vocab"])
    other = toks.copy()
    other[:40] = (other[:40] + 1) % cfg["vocab"]
    oracle = go.Model(cfg, w)
    ref, ref_other = oracle.forward(toks)[0], oracle.forward(other)[0]
    assert tl.rel_err(ref_other[-1], ref[-1]) > 1e-3, "the construction does not carry the first tokens to the end"
    m = make(cfg, w)
    tl.assert_close(run_whole(m, toks), ref, "float32")
    tl.assert_close(run_cut(m, toks, [2, 4, 100, 101, 103, 200]), ref, "float32")
    tl.assert_close(run_cut(m, toks, range(200, n)), ref, "float32")
    m.close()


def test_first_tokens_and_single_token_sequences():
    cfg = full_cfg(loop={"start": 0, "stop": 4, "times": 2}, taps=5)
    w = gl.weights(cfg, seed=12)
    oracle = go.Model(cfg, w)
    m = make(cfg, w)
    for n in (1, 2, 3, 6):
        toks = gl.tokens(50 + n, n, cfg["vocab"])
        ref = oracle.forward(toks)[0]
        tl.assert_close(run_whole(m, toks), ref, "float32")
        tl.assert_close(run_cut(m, toks, range(1, n)), ref, "float32")
    m.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = full_cfg(loop={"start": 1, "stop": 2, "times": 2})
    w = gl.weights(cfg, seed=13)
    toks = gl.tokens(60, 200, cfg["vocab"])
    ref = go.Model(cfg, w).forward(toks)[0]
    m = make(cfg, w, dtype, page_tokens=8)
    got = run_cut(m, toks, range(8, 200))
    tl.assert_close(got, ref, dtype)
    m.close()


def test_larger_odd_sizes_take_the_tiled_products():
    """Sizes that are not multiples of the kernels' tiles and vectors, enough rows for grouped products, a delta-rule state that
    fills a thread's registers, a window of several key tiles."""
    cfg = gl.config([gl.parallel_layer(heads=6, kv_heads=3, dim=20, vdim=10, window=150, rot_dims=14, width=45, blocks=5, conv=4, mlp=gl.moe_mlp(ff=36, experts=6, top=2)),
                     gl.delta_layer(heads=2, kv_heads=1, dim=128, vdim=128, conv=3, decay_rank=10, gate_rank=3, mlp=gl.moe_mlp(ff=100, experts=3, top=2))],
                    vocab=203, width=76, taps=2)
    w = gl.weights(cfg, seed=14)
    toks = gl.tokens(61, 220, cfg["vocab"])
    ref = go.Model(cfg, w).forward(toks)[0]
    for dtype in ("float32", "bfloat16"):
        m = make(cfg, w, dtype)
        tl.assert_close(run_whole(m, toks), ref, dtype, dtype)
        tl.assert_close(run_cut(m, toks, [7, 140, 141, 215]), ref, dtype, dtype)
        m.close()


def test_greedy_and_sampled_generation():
    cfg = full_cfg(loop={"start": 1, "stop": 3, "times": 2})
    w = gl.weights(cfg, seed=15, embed_std=0.5)
    oracle = go.Model(cfg, w)
    prompts = [gl.tokens(70, 9, cfg["vocab"]), gl.tokens(71, 2, cfg["vocab"]), gl.tokens(72, 30, cfg["vocab"])]
    m = make(cfg, w, max_step_tokens=16)
    total = m.free_tokens()
    got = m.generate(prompts, 12)
    for p, g in zip(prompts, got):
        lg, st = oracle.forward(p)
        for t in range(12):
            order = np.argsort(-lg[-1])
            if lg[-1][order[0]] - lg[-1][order[1]] < 1e-3 * np.abs(lg[-1]).max():
                break  # a near tie: fp32 and fp64 may differ from here on
            assert g[t] == order[0], (t, g, order[:3])
            lg, st = oracle.forward([int(g[t])], st)
    assert m.free_tokens() == total  # generate gave every slot and page back
    a = m.generate(prompts, 10, temp=2.0, seed=3)
    assert np.array_equal(a, m.generate(prompts, 10, temp=2.0, seed=3)) and not np.array_equal(a, m.generate(prompts, 10, temp=2.0, seed=4))
    assert np.array_equal(m.generate(prompts, 4, temp=1e-3, seed=1), got[:, :4])
    m.close()


def _checkpoint(tmp_path, cfg, w):
    """A checkpoint folder as it comes from elsewhere: the inner sizes of the two-step projections only in the tensor shapes."""
    cfg = json.loads(json.dumps(cfg))
    for e in cfg["layers"]:
        e["mixer"].pop("decay_rank", None)
        e["mixer"].pop("gate_rank", None)
    d = tmp_path / "ckpt"
    os.makedirs(d, exist_ok=True)
    with open(d / "config.json", "w") as f:
        json.dump(cfg, f)
    weights_io.write_safetensors(str(d / "model.safetensors"), w)
    return str(d)


def test_checkpoint_folder_through_registry_host_program_and_trace_replay(tmp_path):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = full_cfg(loop={"start": 1, "stop": 3, "times": 2})
    w = gl.weights(cfg, seed=16, embed_std=0.5)
    path = _checkpoint(tmp_path, cfg, w)
    prompts = [gl.tokens(80, 11, cfg["vocab"]), gl.tokens(81, 4, cfg["vocab"])]
    m = models.load_model(path, dtype="float32", max_tokens=256, max_seqs=4)
    assert isinstance(m, lm.LayeredLM) and m.config.architecture == "Gupizen"
    want = m.generate(prompts, 9)
    ref = go.Model(cfg, w).forward(prompts[0])[0]
    s = m.open()
    tl.assert_close(m.step([(s, prompts[0], list(range(11)))]), ref, "float32")
    m.close()
    exe = os.path.join(root, "zig_gpt2_amd", "bin", "zgpt2_main")
    arg = ";".join(",".join(str(int(t)) for t in p) for p in prompts)
    out = subprocess.run([exe, "lm", path, arg, "9", "--dtype", "float32"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    got = np.array([[int(t) for t in line.split()] for line in out.stdout.strip().splitlines()])
    assert np.array_equal(got, want)
    a, b = [int(t) for t in prompts[0]], [int(t) for t in prompts[1]]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [5]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[6:9], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b, "want": [0, 3]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[9:10], "want": [0]}], "end": []},
             {"step": 4, "entries": [{"id": "a", "tokens": a[10:11], "want": [0]}], "end": ["a"]},
             {"step": 5, "entries": [{"id": "c", "tokens": a, "want": [10]}], "end": ["c"]}]
    outdir = tmp_path / "out"
    run = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32", "--out", str(outdir),
                          "--max-tokens", "64"], input="\n".join(json.dumps(x) for x in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(6)]
    refb = go.Model(cfg, w).forward(prompts[1])[0]
    rd = lambda i: np.fromfile(str(outdir / f"{i}.f32"), dtype="<f4").reshape(-1, cfg["vocab"])  # noqa: E731
    assert not (outdir / "1.f32").exists()
    tl.assert_close(rd(0), ref[5:6], "float32")
    tl.assert_close(rd(2), refb[[0, 3]], "float32")
    tl.assert_close(rd(3), ref[9:10], "float32")
    tl.assert_close(rd(4), ref[10:11], "float32")
    tl.assert_close(rd(5), ref[10:11], "float32")


def test_scheduler_serves_more_requests_than_slots():
    """Continuous batching: seven requests of unequal lengths on two slots — every request's tokens equal its generation alone,
    slots and pages go round, also the pages that the windows leave behind while a request is still running."""
    cfg = full_cfg(loop={"start": 0, "stop": 2, "times": 2})
    w = gl.weights(cfg, seed=18, embed_std=0.5)
    m = make(cfg, w, max_tokens=128, max_seqs=2, page_tokens=8)
    reqs = [(gl.tokens(90 + i, n, cfg["vocab"]), k) for i, (n, k) in enumerate([(30, 6), (3, 9), (17, 2), (1, 12), (41, 5), (8, 8), (2, 1)])]
    alone = [m.generate([p], k)[0] for p, k in reqs]
    total = m.free_tokens()
    sch = lm.Scheduler(m, portion=16)
    ids = [sch.submit(p, k) for p, k in reqs]
    out = sch.run()
    for rid, want in zip(ids, alone):
        assert np.array_equal(out[rid], want), (rid, out[rid], want)
    assert m.free_tokens() == total and sch._reserved == 0
    assert sch.steps < sum(-(-len(p) // 16) + k for p, k in reqs)  # requests shared steps
    m.close()

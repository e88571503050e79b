"""The layered-model tier (zg_lm_*, zig_gpt2_amd/lm.py) against the float64 oracle of tests/lm_oracle.py: every mechanism alone,
whole prompts against portions and token-by-token decoding, ragged batches, slot and page reuse, far keys and page borders,
other sizes, and generation through the library's own entry point."""
import numpy as np
import pytest

import lm_oracle
import lm_testlib as tl
from zig_gpt2_amd import lm

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
    "hgrn2": [tl.hgrn2_layer()],
    "hgrn2_wide": [tl.hgrn2_layer(heads=1, dim=40, vdim=72)],  # more key channels than one lane holds, columns beyond a wave
    "latent": [tl.latent_layer()],
    "latent_plain_rotary": [tl.latent_layer(scaling=None, rot_dim=12, rot_dims=8)],  # part of the rotary part passes unrotated
    "latent_one_head": [tl.latent_layer(heads=1, dim=8, vdim=8, rot_dim=4, kv_rank=72, q_rank=8)],  # more than 64 cached dimensions
    "dense": [tl.hgrn2_layer(mlp=tl.dense_mlp())],
    "moe": [tl.hgrn2_layer(mlp=tl.moe_mlp())],
    "moe_top1": [tl.hgrn2_layer(mlp=tl.moe_mlp(ff=20, experts=3, top=1))],
    "moe_all": [tl.hgrn2_layer(mlp=tl.moe_mlp(ff=8, experts=4, top=4))],
    "moe_many": [tl.hgrn2_layer(mlp=tl.moe_mlp(ff=8, experts=70, top=3))],  # more experts than a wave has lanes
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_alone(name, dtype):
    cfg = tl.config(SINGLE[name])
    w = tl.weights(cfg, seed=sum(map(ord, name)))
    toks = tl.tokens(1, 37, cfg["vocab"])
    ref, _, ref_tr = lm_oracle.Model(cfg, w).forward(toks, want_layers=True)
    m = make(cfg, w, dtype)
    got, tr = run_whole(m, toks, trace=True)
    tl.assert_close(tr, ref_tr, dtype, "residual stream")
    tl.assert_close(got, ref, dtype, "logits")
    # the same prompt token by token: the decode kernels, state carried by the slot
    step = run_cut(m, toks, range(1, len(toks)))
    tl.assert_close(step, ref, dtype, "decoded")
    m.close()


def full_cfg(**kw):
    return tl.config([tl.hgrn2_layer(mlp=tl.dense_mlp()), tl.latent_layer(mlp=tl.moe_mlp()), tl.latent_layer(heads=2, dim=8, vdim=40, kv_rank=24, q_rank=16, rot_dim=16, mlp=None),
                      tl.hgrn2_layer(heads=3, dim=8, vdim=16, mlp=tl.moe_mlp(experts=7, top=3))], **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_several_sizes(dtype):
    cfg = full_cfg(loop={"start": 1, "stop": 3, "times": 2})
    w = tl.weights(cfg, seed=5)
    toks = tl.tokens(2, 90, cfg["vocab"])
    ref, _ = lm_oracle.Model(cfg, w).forward(toks)
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
    for loop in (None, {"start": 0, "stop": 4, "times": 3}, {"start": 2, "stop": 3, "times": 2}, {"start": 0, "stop": 1, "times": 1}):
        cfg = full_cfg(loop=loop)
        w = tl.weights(cfg, seed=6)
        toks = tl.tokens(3, 21, cfg["vocab"])
        ref, _, ref_tr = lm_oracle.Model(cfg, w).forward(toks, want_layers=True)
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
    w = tl.weights(cfg, seed=7)
    oracle = lm_oracle.Model(cfg, w)
    lens = [41, 3, 17, 1]
    prompts = [tl.tokens(10 + i, n, cfg["vocab"]) for i, n in enumerate(lens)]
    refs = [oracle.forward(p)[0] for p in prompts]
    m = make(cfg, w, dtype, page_tokens=4)
    seqs = [m.open() for _ in prompts]
    # step 1: unequal first portions of all four; step 2: the rest of the long ones beside single decoded tokens
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
    more = [tl.tokens(20 + i, 6, cfg["vocab"]) for i in range(3)]
    alone = [oracle.forward(np.concatenate([prompts[i], more[i]]))[0][len(prompts[i]):] for i in range(3)]
    rows = [m.step([(seqs[i], [more[i][t]], [0]) for i in range(3)]) for t in range(6)]
    for i in range(3):
        tl.assert_close(np.stack([r[i] for r in rows]), alone[i], dtype, i)
    m.close()


def test_slots_and_pages_are_reused():
    cfg = full_cfg()
    w = tl.weights(cfg, seed=8)
    oracle = lm_oracle.Model(cfg, w)
    m = make(cfg, w, max_tokens=64, max_seqs=2, page_tokens=4)
    total = m.free_tokens()
    a, b = tl.tokens(30, 33, cfg["vocab"]), tl.tokens(31, 26, cfg["vocab"])
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
        sb = m.open()
        got = m.step([(sb, b, list(range(len(b))))])
        tl.assert_close(got, rb, "float32", rnd)  # nothing of the slot's former sequence is left
        with pytest.raises(Exception):
            m.step([(sa, a, [])])  # more tokens than the cache has pages for
        assert m.seq_len(sa) == 33 and m.seq_len(sb) == 26
        m.close_seq(sa)
        m.close_seq(sb)
        assert m.free_tokens() == total
    m.close()


def test_far_keys_stand_out():
    """A sharp softmax (large score factor) puts nearly all weight on single keys, many of them far back and across page
    borders: a key that is lost, shifted by one or read from a wrong page changes the result by its whole value."""
    lay = tl.latent_layer(heads=2, dim=16, vdim=16, rot_dim=8, kv_rank=32, q_rank=32, scale=6.0)
    cfg = tl.config([lay], width=32)
    w = tl.weights(cfg, seed=9)
    n = 300
    toks = tl.tokens(40, n, cfg["vocab"])
    oracle = lm_oracle.Model(cfg, w)
    ref, _ = oracle.forward(toks)
    # how peaked and how far: recompute the attention weights of the oracle's own layer
    x = oracle.w["embed"][toks]
    h = lm_oracle.norm_around_zero(x, oracle.w["l0.norm1"], oracle.eps)
    h, _ = lm_oracle.token_shift(h, oracle.w["l0.shift"], None)
    att = lm_oracle.attention_weights(h, oracle.w, "l0.mix.", lay["mixer"], oracle.eps, np.arange(n))
    top = att.max(axis=-1)  # [heads, queries]
    far = np.arange(n)[None, :] - att.argmax(axis=-1)
    assert (top[:, 200:] > 0.9).mean() > 0.5 and (far[:, 200:] > 100).sum() > 20, "the construction does not make far keys stand out"
    m = make(cfg, w, page_tokens=16)
    assert tl.rel_err(run_whole(m, toks), ref) < 2e-4
    assert tl.rel_err(run_cut(m, toks, [15, 16, 17, 150, 255, 256, 257]), ref) < 2e-4
    # decoded one by one behind a long prompt
    got = run_cut(m, toks, range(270, n))
    assert tl.rel_err(got, ref) < 2e-4
    m.close()


def test_recurrence_remembers_far_tokens():
    """Lower bounds close to one: the recurrent state forgets slowly, so the first tokens still weigh in hundreds of tokens
    later — a state that is lost or reset between portions shows."""
    cfg = tl.config([tl.hgrn2_layer(heads=2, dim=16, vdim=16)], width=32)
    w = tl.weights(cfg, seed=10, lower=(0.97, 0.999))
    n = 260
    toks = tl.tokens(41, n, cfg["vocab"])
    other = toks.copy()
    other[:8] = (other[:8] + 1) % cfg["vocab"]
    oracle = lm_oracle.Model(cfg, w)
    ref, ref_other = oracle.forward(toks)[0], oracle.forward(other)[0]
    assert tl.rel_err(ref_other[-1], ref[-1]) > 1e-3, "the construction does not carry the first tokens to the end"
    m = make(cfg, w)
    tl.assert_close(run_whole(m, toks), ref, "float32")
    tl.assert_close(run_cut(m, toks, [2, 4, 100, 101, 103, 200]), ref, "float32")
    tl.assert_close(run_cut(m, toks, range(200, n)), ref, "float32")
    m.close()


def test_first_tokens_and_single_token_sequences():
    cfg = full_cfg(loop={"start": 0, "stop": 4, "times": 2})
    w = tl.weights(cfg, seed=11)
    oracle = lm_oracle.Model(cfg, w)
    m = make(cfg, w)
    for n in (1, 2, 3):
        toks = tl.tokens(50 + n, n, cfg["vocab"])
        ref = oracle.forward(toks)[0]
        tl.assert_close(run_whole(m, toks), ref, "float32")
        tl.assert_close(run_cut(m, toks, range(1, n)), ref, "float32")
    m.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = full_cfg(loop={"start": 1, "stop": 2, "times": 2})
    w = tl.weights(cfg, seed=12)
    toks = tl.tokens(60, 200, cfg["vocab"])
    ref = lm_oracle.Model(cfg, w).forward(toks)[0]
    m = make(cfg, w, dtype, page_tokens=8)
    got = run_cut(m, toks, range(8, 200))
    tl.assert_close(got, ref, dtype)
    m.close()


def test_larger_odd_sizes_take_the_tiled_products():
    """Sizes that are not multiples of the kernels' tiles and vectors, and enough rows for the large tiles and grouped products."""
    cfg = tl.config([tl.hgrn2_layer(heads=3, dim=20, vdim=28, mlp=tl.moe_mlp(ff=36, experts=6, top=2)),
                     tl.latent_layer(heads=5, dim=12, vdim=20, rot_dim=6, rot_dims=6, kv_rank=52, q_rank=44, mlp=tl.dense_mlp(ff=100))], vocab=203, width=76)
    w = tl.weights(cfg, seed=13)
    toks = tl.tokens(61, 150, cfg["vocab"])
    ref = lm_oracle.Model(cfg, w).forward(toks)[0]
    for dtype in ("float32", "bfloat16"):
        m = make(cfg, w, dtype)
        tl.assert_close(run_whole(m, toks), ref, dtype, dtype)
        tl.assert_close(run_cut(m, toks, [7, 140, 141]), ref, dtype, dtype)
        m.close()


def test_large_tiles_on_small_shapes(monkeypatch):
    """The 128 x 128 tiles (taken by themselves only from thousands of rows) on shapes with ragged edges, grouped products included."""
    monkeypatch.setenv("ZGPT2_LM_GEMM_TILE", "128")
    cfg = tl.config([tl.hgrn2_layer(heads=3, dim=20, vdim=28, mlp=tl.moe_mlp(ff=36, experts=3, top=2)),
                     tl.latent_layer(heads=2, dim=12, vdim=20, rot_dim=6, kv_rank=52, q_rank=44, mlp=tl.dense_mlp(ff=150))], vocab=203, width=76)
    w = tl.weights(cfg, seed=17)
    toks = tl.tokens(62, 300, cfg["vocab"])
    ref = lm_oracle.Model(cfg, w).forward(toks)[0]
    for dtype in ("float32", "bfloat16"):
        m = make(cfg, w, dtype)
        tl.assert_close(run_whole(m, toks), ref, dtype, dtype)
        m.close()


def test_long_rows_in_decode_steps():
    """Feed-forward widths beyond 1536: decode steps multiply their down-projections with K split over the waves of a workgroup
    (one width a multiple of the 16-byte pieces, one not) alone and as a batch of two; a batch of three takes the general kernel."""
    cfg = tl.config([tl.hgrn2_layer(mlp=tl.dense_mlp(ff=1620)), tl.latent_layer(mlp=tl.dense_mlp(ff=1544))])
    w = tl.weights(cfg, seed=19)
    oracle = lm_oracle.Model(cfg, w)
    toks = [tl.tokens(63 + i, 14, cfg["vocab"]) for i in range(3)]
    refs = [oracle.forward(t)[0] for t in toks]
    for dtype in ("float32", "bfloat16"):
        m = make(cfg, w, dtype)
        tl.assert_close(run_cut(m, toks[0], range(1, 14)), refs[0], dtype, dtype)
        for nb in (2, 3):
            seqs = [m.open() for _ in range(nb)]
            rows = [m.step([(s, [t[i]], [0]) for s, t in zip(seqs, toks)]) for i in range(14)]
            for b in range(nb):
                tl.assert_close(np.stack([r[b] for r in rows]), refs[b], dtype, (dtype, nb, b))
            for s in seqs:
                m.close_seq(s)
        m.close()


def test_rows_wider_than_the_register_kernels():
    """A width beyond what the one-round-trip norm kernels hold in registers: the general norm kernels and the unfused pass tail."""
    cfg = tl.config([tl.hgrn2_layer(heads=1, dim=8, vdim=8, mlp=tl.moe_mlp(ff=8, experts=3, top=2)),
                     tl.latent_layer(heads=1, dim=8, vdim=8, rot_dim=4, kv_rank=16, q_rank=8, mlp=tl.dense_mlp(ff=16))], vocab=61, width=4100)
    w = tl.weights(cfg, seed=20)
    toks = tl.tokens(64, 12, cfg["vocab"])
    ref = lm_oracle.Model(cfg, w).forward(toks)[0]
    m = make(cfg, w, "float32", max_tokens=64, max_seqs=2)
    tl.assert_close(run_whole(m, toks), ref, "float32")
    tl.assert_close(run_cut(m, toks, [2, 3, 4, 5, 6, 7, 8, 9]), ref, "float32")
    m.close()


def test_greedy_and_sampled_generation():
    cfg = full_cfg(loop={"start": 1, "stop": 3, "times": 2})
    w = tl.weights(cfg, seed=14, head_std=1.0)
    oracle = lm_oracle.Model(cfg, w)
    prompts = [tl.tokens(70, 9, cfg["vocab"]), tl.tokens(71, 2, cfg["vocab"]), tl.tokens(72, 30, cfg["vocab"])]
    m = make(cfg, w, max_step_tokens=16)
    got = m.generate(prompts, 12)
    for p, g in zip(prompts, got):
        lg, st = oracle.forward(p)
        for t in range(12):
            order = np.argsort(-lg[-1])
            if lg[-1][order[0]] - lg[-1][order[1]] < 1e-3 * np.abs(lg[-1]).max():
                break  # a near tie: fp32 and fp64 may differ from here on
            assert g[t] == order[0], (t, g, order[:3])
            lg, st = oracle.forward([int(g[t])], st)
    assert m.free_tokens() == (512 // 64 + 4) * 64  # generate gave every slot and page back
    a = m.generate(prompts, 10, temp=0.9, seed=3)
    assert np.array_equal(a, m.generate(prompts, 10, temp=0.9, seed=3)) and not np.array_equal(a, m.generate(prompts, 10, temp=0.9, seed=4))
    assert a.min() >= 0 and a.max() < cfg["vocab"] and not np.array_equal(a, got[:, :10])
    # a nearly zero temperature draws the greedy token
    assert np.array_equal(m.generate(prompts, 4, temp=1e-3, seed=1), got[:, :4])
    m.close()


def test_errors_are_reported():
    cfg = full_cfg()
    w = tl.weights(cfg, seed=15)
    m = lm.LayeredLM(lm.LMConfig.from_json(cfg), dtype="float32", max_tokens=64, max_seqs=2)
    with pytest.raises(Exception):
        m.load_weights({"nope": np.zeros(3, np.float32)})
    with pytest.raises(Exception):
        m.load_weights({"embed": np.zeros((3, 3), np.float32)}, strict=False)
    s = m.open()
    with pytest.raises(Exception):
        m.step([(s, [1, 2], [0])])  # weights missing
    m.load_weights(w)
    with pytest.raises(Exception):
        m.step([(s, [1, cfg["vocab"]], [0])])
    with pytest.raises(Exception):
        m.step([(s, [1, 2], [2])])
    with pytest.raises(Exception):
        m.step([(s + 1, [1], [0])])
    with pytest.raises(Exception):
        m.step([(s, [1], [0]), (s, [2], [0])])
    assert m.seq_len(s) == 0
    assert m.step([(s, [1, 2], [])]).shape == (0, cfg["vocab"]) and m.seq_len(s) == 2
    m.close()
    bad = full_cfg()
    bad["layers"][1]["mixer"]["rot"]["dims"] = 7
    with pytest.raises(Exception):
        lm.LayeredLM(lm.LMConfig.from_json(bad), max_tokens=64)


def _checkpoint(tmp_path, cfg, w):
    import json

    from zig_gpt2_amd import weights_io

    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    extra = dict(w)
    extra["positions.table"] = np.arange(6, dtype=np.int32)  # not a tensor of the configuration: every front end leaves it alone
    weights_io.write_safetensors(str(d / "model.safetensors"), extra)
    return str(d)


def test_checkpoint_folder_through_registry_host_program_and_trace_replay(tmp_path):
    """One checkpoint folder, three front ends: models.load_model (the registry picks the class from config.json), the C++ host
    program's `lm` command, and the trace replay program — all on the library's step / generate."""
    import json
    import os
    import subprocess
    import sys

    from zig_gpt2_amd import models

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = full_cfg(loop={"start": 1, "stop": 3, "times": 2})
    w = tl.weights(cfg, seed=16, head_std=1.0)
    path = _checkpoint(tmp_path, cfg, w)
    prompts = [tl.tokens(80, 11, cfg["vocab"]), tl.tokens(81, 4, cfg["vocab"])]
    m = models.load_model(path, dtype="float32", max_tokens=256, max_seqs=4)
    assert isinstance(m, lm.LayeredLM)
    want = m.generate(prompts, 9)
    ref = lm_oracle.Model(cfg, w).forward(prompts[0])[0]
    s = m.open()
    tl.assert_close(m.step([(s, prompts[0], list(range(11)))]), ref, "float32")
    m.close()
    exe = os.path.join(root, "zig_gpt2_amd", "bin", "zgpt2_main")
    arg = ";".join(",".join(str(int(t)) for t in p) for p in prompts)
    out = subprocess.run([exe, "lm", path, arg, "9", "--dtype", "float32"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    got = np.array([[int(t) for t in line.split()] for line in out.stdout.strip().splitlines()])
    assert np.array_equal(got, want)
    bad = subprocess.run([exe, "lm", path, "1,100000", "2"], capture_output=True, text=True, timeout=120)
    assert bad.returncode != 0 and "vocabulary" in bad.stderr
    # trace replay: a prompt in two portions and two decoded tokens, a second request between them, the first one ended and its
    # slot taken again
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
    refb = lm_oracle.Model(cfg, w).forward(prompts[1])[0]
    rd = lambda i: np.fromfile(str(outdir / f"{i}.f32"), dtype="<f4").reshape(-1, cfg["vocab"])  # noqa: E731
    assert not (outdir / "1.f32").exists()
    tl.assert_close(rd(0), ref[5:6], "float32")
    tl.assert_close(rd(2), refb[[0, 3]], "float32")
    tl.assert_close(rd(3), ref[9:10], "float32")
    tl.assert_close(rd(4), ref[10:11], "float32")
    tl.assert_close(rd(5), ref[10:11], "float32")


def test_scheduler_serves_more_requests_than_slots():
    """Continuous batching: seven requests of unequal lengths on two slots and a cache that holds about two of them — every
    request's tokens equal its generation alone, slots and pages go round."""
    cfg = full_cfg(loop={"start": 0, "stop": 2, "times": 2})
    w = tl.weights(cfg, seed=18, head_std=1.0)
    m = make(cfg, w, max_tokens=128, max_seqs=2, page_tokens=8)
    reqs = [(tl.tokens(90 + i, n, cfg["vocab"]), k) for i, (n, k) in enumerate([(30, 6), (3, 9), (17, 2), (1, 12), (41, 5), (8, 8), (2, 1)])]
    alone = [m.generate([p], k)[0] for p, k in reqs]
    total = m.free_tokens()
    sch = lm.Scheduler(m, portion=16)
    ids = [sch.submit(p, k) for p, k in reqs]
    out = sch.run()
    for rid, want in zip(ids, alone):
        assert np.array_equal(out[rid], want), (rid, out[rid], want)
    assert m.free_tokens() == total and sch._reserved == 0
    assert sch.steps < sum(-(-len(p) // 16) + k for p, k in reqs)  # requests shared steps
    with pytest.raises(Exception):
        lm.Scheduler(m).submit([], 3)
    m.close()

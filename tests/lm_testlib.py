"""Small random layered-model configurations and weights for the tests (bf16-representable values, so that the float64 oracle
and the bf16-storage device path see the same numbers)."""
import numpy as np

from zig_gpt2_amd.synth import round_bf16


def hgrn2_layer(heads=2, dim=16, vdim=24, mlp=None):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}, "mlp": mlp}


def latent_layer(heads=3, dim=16, vdim=24, rot_dim=8, kv_rank=40, q_rank=48, scale=0.2, rot_dims=None, base=10000.0, scaling="default", mlp=None):
    rot = {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}
    if scaling == "default":
        scaling = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "rot_dim": rot_dim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale, "rot": rot},
            "mlp": mlp}


def dense_mlp(ff=96):
    return {"kind": "dense", "ff": ff}


def moe_mlp(ff=24, experts=5, top=2):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(layers, vocab=97, width=48, loop=None, eps=1e-5):
    return {"architecture": "Tokosun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers, "loop": loop}


def weights(cfg, seed=0, std=None, lower=(0.0, 1.0), head_std=None):
    """Random tensors for every name of the configuration.  std: matrices ~ N(0, std^2), default 1 / sqrt(fan_in) so that the
    activations keep their size from layer to layer; lower: range of the recurrence's lower bounds."""
    from zig_gpt2_amd import lm

    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in lm.LMConfig.from_json(cfg).tensor_shapes().items():
        leaf = name.split(".")[-1]
        if len(shape) == 2:
            s = std if std is not None else 1.0 / np.sqrt(shape[1])
            if name == "embed":
                s = 1.0
            if name == "head" and head_std is not None:
                s = head_std
            a = rng.normal(0.0, s, shape)
        elif leaf == "lower":
            a = rng.uniform(lower[0], lower[1], shape)
        elif leaf == "shift":
            a = rng.uniform(0.0, 1.0, shape)
        elif name.endswith("mix.norm") or name.endswith("dq.norm") or name.endswith("dkv.norm"):
            a = 1.0 + rng.normal(0.0, 0.1, shape)
        elif leaf == "correction":
            a = rng.normal(0.0, 0.05, shape)
        elif leaf == "b":
            a = rng.normal(0.0, 0.5, shape)
        else:  # norm offsets around zero
            a = rng.normal(0.0, 0.1, shape)
        out[name] = round_bf16(a.astype(np.float32)).reshape(shape)
    return out


def tokens(seed, n, vocab):
    return np.random.default_rng(1000 + seed).integers(0, vocab, n).astype(np.int32)


def rel_err(got, want):
    """Largest difference relative to the largest expected magnitude."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


TOL = {"float32": 3e-5, "bfloat16": 4e-2}


def assert_close(got, want, dtype, what=""):
    """float32: every element within TOL of the largest expected magnitude.  bfloat16: rounding of an activation can flip a
    router's close call or a greedy near-tie at a single token, which moves that token's row (and, fading, the rows behind it)
    by far more than rounding does — so nine rows in ten must be within TOL and the typical row well inside; the sharp
    statement about every row is the float32 one."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    scale = max(np.abs(want).max(), 1e-30)
    rows = np.abs(got - want).reshape(-1, want.shape[-1]).max(axis=-1) / scale
    assert np.isfinite(rows).all(), what
    if dtype == "float32":
        assert rows.max() < TOL[dtype], (what, float(rows.max()), int(rows.argmax()))
    elif rows.size < 10:  # too few rows for a statement about most of them
        assert np.median(rows) < TOL[dtype], (what, float(np.median(rows)))
    else:
        assert np.quantile(rows, 0.9) < TOL[dtype] and np.median(rows) < TOL[dtype] / 3, (what, float(np.quantile(rows, 0.9)), float(np.median(rows)))

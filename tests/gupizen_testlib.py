"""Small random Gupizen configurations and weights for the tests (bf16-representable values, so that the float64 oracle and
the bf16-storage device path see the same numbers)."""
import numpy as np

from zig_gpt2_amd.synth import round_bf16

BANDS = {"factor": 4.0, "low": 1.0, "high": 8.0, "original": 64}  # with base 100 and 8 rotated dims: one pair per band


def parallel_layer(heads=4, kv_heads=2, dim=12, vdim=8, window=7, scale=0.3, rot_dims=8, base=100.0, scaling="default", width=20, blocks=2, conv=3,
                   mlp=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling == "default":
        scaling = dict(BANDS)
    if scaling:
        rot["scaling"] = scaling
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if window:
        left["mask"] = {"size": window}
    return {"type": "parallel", "mixer": {"left": left, "right": {"width": width, "blocks": blocks, "conv": conv}}, "mlp": mlp}


def delta_layer(heads=4, kv_heads=2, dim=8, vdim=12, conv=4, decay_rank=6, gate_rank=5, mlp=None):
    return {"type": "channel_delta",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "decay_rank": decay_rank, "gate_rank": gate_rank},
            "mlp": mlp}


def moe_mlp(ff=24, experts=5, top=2):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(layers, vocab=97, width=48, loop=None, eps=1e-5, taps=3, embed_scale=0.7):
    return {"architecture": "Gupizen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers, "loop": loop,
            "canon": {"taps": taps}, "embedding": {"scale": embed_scale}}


def weights(cfg, seed=0, lam_mean=-1.0, a_log_mean=-1.0, sink_mean=0.0, embed_std=1.0):
    """Random tensors for every name of the configuration.  Matrices ~ N(0, 1 / fan_in).  lam_mean / a_log_mean: how fast the
    recurrent unit / the delta rule forget (very negative: hardly at all); sink_mean: how much weight the sinks draw."""
    from zig_gpt2_amd import lm

    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in lm.LMConfig.from_json(cfg).tensor_shapes().items():
        leaf = name.split(".")[-1]
        two = ".".join(name.split(".")[-2:])
        if leaf == "talk":
            a = np.eye(shape[0]) + rng.normal(0.0, 0.25, shape)
        elif leaf in ("canon1", "canon2") or two in ("q.conv", "k.conv", "v.conv", "right.conv"):
            a = rng.normal(0.0, 0.4, shape)
        elif leaf in ("ra", "ri"):
            a = rng.normal(0.0, 1.0 / np.sqrt(shape[-1]), shape)
        elif name == "embed":
            a = rng.normal(0.0, embed_std, shape)
        elif len(shape) == 2 and leaf != "b" or two == "mix.b":
            a = rng.normal(0.0, 1.0 / np.sqrt(shape[1]), shape)
        elif leaf == "sink":
            a = rng.normal(sink_mean, 1.0, shape)
        elif leaf == "lam":
            a = rng.normal(lam_mean, 0.5, shape)
        elif leaf == "A_log":
            a = rng.normal(a_log_mean, 0.3, shape)
        elif leaf in ("b", "dt_bias"):
            a = rng.normal(0.0, 0.4, shape)
        elif two in ("mix.norm", "left.out", "right.out"):
            a = 1.0 + rng.normal(0.0, 0.1, shape)
        else:  # norm offsets around zero
            a = rng.normal(0.0, 0.1, shape)
        out[name] = round_bf16(a.astype(np.float32)).reshape(shape)
    return out


def tokens(seed, n, vocab):
    return np.random.default_rng(2000 + seed).integers(0, vocab, n).astype(np.int32)

"""Shared pieces of the Sanevik tests: small configurations of the design (sizes of the tests' own making: a width that is
no multiple of 32, head sizes on and off the matrix cores' shapes, rotated parts shorter than a head, grouped and ungrouped
key/value heads, one tap and five, loops over a prefix, the middle or all of the layers, one pass and three, no loop at
all, routers that take one expert or several), random checkpoints written as a model directory.  The replay helper that
feeds sequences to the engine's row-step path in a given cut is the one of gazutar_harness (it is not specific to a
model)."""
import json
import os
import tempfile

import torch

from gazutar_harness import F32_BAR, Replay, rel_err, row_errs, tokens_of  # noqa: F401 (re-exported)

BF16_MEDIAN, BF16_ROW = 2e-2, 6e-2


def assert_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what="") -> None:
    """float32 mode: every row within F32_BAR (row-wise rms difference / rms of the expected row).  bfloat16 mode: the
    rounding of activations on their way into the matrix cores gives these stacks about 1e-2 per row, and a router's
    near-tie that falls the other way replaces an expert for that token (and, through the recurrent state, moves later
    rows): the median row within BF16_MEDIAN, at most a quarter of the rows over BF16_ROW.  Position-exact faults are the
    float32 runs' business."""
    e = row_errs(got, want)
    if dtype == "float32":
        assert float(e.max()) <= F32_BAR, (what, float(e.max()), int(e.argmax()))
    else:
        off = int((e > BF16_ROW).sum())
        assert float(e.median()) <= BF16_MEDIAN and off <= max(1, e.numel() // 4), (what, float(e.median()), off, e.numel())


def rot(dims, base=10000.0, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling:
        r["scaling"] = scaling
    return r


LONG = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}   # a ramp that falls inside a 24-channel rotation


def attention(heads=6, kv_heads=3, dim=24, vdim=20, window=17, scale=0.3, dims=16, scaling=LONG, base=10000.0):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window}, "scale": scale,
                      "rot": rot(dims, base, scaling)}}


def parallel(heads=4, kv_heads=2, dim=16, vdim=24, window=13, scale=0.4, softcap=3.0, conv=3, dims=8,
             r_heads=3, r_dim=20, r_vdim=12, r_dims=12, decay=None, left_scale=0.7, right_scale=1.2):
    decay = decay or [1 - 2.0 ** -(2 + h) for h in range(r_heads)]
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
                               "scale": scale, "softcap": softcap, "conv": conv, "rot": rot(dims)},
                      "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "decay": decay, "rot": rot(r_dims, 500.0)},
                      "left_scale": left_scale, "right_scale": right_scale}}


def moe(ff=40, experts=7, top=3, limit=1.0):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


def config(layers, width=80, vocab=97, loop=(0, 0, 0), eps=1e-5):
    cfg = {"architecture": "Sanevik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop[2]:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# the parallel layer first and again inside the loop, a layer without feed-forward, grouped and ungrouped heads, a loop over
# the middle layers (three passes), head sizes on and off the matrix cores' shapes
MIXED = config([
    with_mlp(parallel(), moe()),
    with_mlp(attention(), moe(ff=24, experts=5, top=1)),
    with_mlp(parallel(heads=2, kv_heads=2, dim=32, vdim=32, window=40, conv=2, dims=32, r_heads=2, r_dim=32, r_vdim=32,
                      r_dims=32), None),
    with_mlp(attention(heads=4, kv_heads=4, dim=32, vdim=16, window=9, dims=32, scaling=None), moe(ff=16, experts=12, top=4)),
    with_mlp(attention(heads=2, kv_heads=1, dim=10, vdim=6, window=200, dims=4), moe()),
], loop=(1, 4, 3))


def write_model_dir(cfg: dict, weights: dict) -> str:
    from safetensors.torch import save_file

    d = tempfile.mkdtemp(prefix="sanevik_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, os.path.join(d, "model.safetensors"))
    return d

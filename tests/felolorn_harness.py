"""Shared pieces of the Felolorn tests: small configurations of the design (sizes of the tests' own making: widths that are
no multiple of 32, key / value / latent sizes that are not whole 16-byte pieces next to ones that are, one tap and five,
one expert group and four), random checkpoints written as a model directory.  The replay helper that feeds sequences to the
engine's row-step path in a given cut is the one of gazutar_harness (it is not specific to a model)."""
import json
import os
import tempfile

import torch

from gazutar_harness import F32_BAR, Replay, rel_err, row_errs, tokens_of  # noqa: F401 (re-exported)

BF16_MEDIAN, BF16_ROW = 2e-2, 6e-2


def assert_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what="") -> None:
    """float32 mode: every row within F32_BAR (row-wise rms difference / rms of the expected row).  bfloat16 mode: the
    rounding of activations on their way into the matrix cores gives these stacks about 1e-2 per row, and a router's
    near-tie that falls the other way moves single rows (and, through the recurrent state, later ones) by tens of percent:
    the median row within BF16_MEDIAN, at most a quarter of the rows over BF16_ROW.  Position-exact faults are the float32
    runs' business."""
    e = row_errs(got, want)
    if dtype == "float32":
        assert float(e.max()) <= F32_BAR, (what, float(e.max()), int(e.argmax()))
    else:
        off = int((e > BF16_ROW).sum())
        assert float(e.median()) <= BF16_MEDIAN and off <= max(1, e.numel() // 4), (what, float(e.median()), off, e.numel())


def latent(heads=3, dim=24, vdim=20, kv_rank=40, q_rank=28, scale=0.15):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale}}


def lightning(heads=3, dim=20, vdim=24, decay=None):
    decay = decay or [0.5 + 0.49 * (h + 1) / heads for h in range(heads)]
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def hgrn2(heads=2, dim=24, vdim=36):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}}


def moe(ff=40, experts=12, top=3, count=4, keep=2):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


def config(layers, width=80, vocab=97, taps=3, scale=7.0, cap=9.0, eps=1e-5):
    return {"architecture": "Felolorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "canon": {"taps": taps},
            "embedding": {"scale": scale}, "logit_softcap": cap, "layers": layers}


# a recurrence first, every mixer, routers with several kept groups / one group / groups of one expert, a layer without
# feed-forward, latent sizes on and off the matrix cores' shapes
MIXED = config([
    with_mlp(hgrn2(), moe()),
    with_mlp(latent(), moe(ff=24, experts=5, top=2, count=1, keep=1)),
    with_mlp(lightning(), None),
    with_mlp(latent(heads=4, dim=16, vdim=32, kv_rank=64, q_rank=48, scale=0.2), moe(ff=32, experts=6, top=2, count=6, keep=3)),
    with_mlp(lightning(heads=2, dim=40, vdim=16), moe(ff=16, experts=8, top=4, count=2, keep=1)),
    with_mlp(hgrn2(heads=5, dim=8, vdim=12), moe()),
])


def write_model_dir(cfg: dict, weights: dict) -> str:
    from safetensors.torch import save_file

    d = tempfile.mkdtemp(prefix="felolorn_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, os.path.join(d, "model.safetensors"))
    return d

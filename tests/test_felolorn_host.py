"""Host-side pieces of the Felolorn integration (no GPU): the configuration reader, the checkpoint name map through the
framework's loader, what a sequence needs in pages and state slots, and the plain statement's own consistency."""
import os

import pytest
import torch

from felolorn_harness import MIXED, config, hgrn2, latent, lightning, moe, with_mlp, write_model_dir
from oracle import felolorn as F


@pytest.fixture(scope="module")
def model_dir():
    return write_model_dir(MIXED, F.random_model(MIXED, seed=1))


def test_config_is_read_from_the_directory(model_dir):
    from nanovllm.config import Config

    c = Config(model_dir, dtype="float32", max_model_len=128, max_num_batched_tokens=128)
    hf = c.hf_config
    assert c.hybrid_state and hf.architectures == ["Felolorn"]
    assert (hf.vocab_size, hf.hidden_size, hf.num_hidden_layers) == (MIXED["vocab"], MIXED["width"], 6)
    assert hf.conv_taps == 3 and hf.embedding_scale == 7.0 and hf.logit_softcap == 9.0 and hf.norm_eps == 1e-5
    assert c.eos == -1 and c.max_model_len == 128


def test_absent_constants_mean_absent_mechanisms():
    from nanovllm.models.felolorn import FelolornConfig

    raw = config([with_mlp(lightning(), None)])
    del raw["embedding"], raw["logit_softcap"]
    c = FelolornConfig(raw)
    assert c.embedding_scale == 1.0 and c.logit_softcap == 0.0


def test_every_tensor_lands_in_a_parameter(model_dir):
    """Load through the framework's loader on the CPU: every parameter is written, merged and stacked ones in the right
    row ranges, the per-head up-projections in their batched layouts, and nothing of the checkpoint is left over."""
    from nanovllm.models.felolorn import FelolornConfig, FelolornForCausalLM
    from nanovllm.utils.loader import load_model
    from safetensors.torch import load_file

    model = FelolornForCausalLM(FelolornConfig.from_dir(model_dir))
    for p in model.parameters():
        p.data.fill_(float("nan"))
    load_model(model, model_dir)
    w = {k: v.float() for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    for name, p in model.named_parameters():
        assert not torch.isnan(p).any(), name
    assert sum(p.numel() for p in model.parameters()) == sum(v.numel() for v in w.values())
    gru, lat, lin = model.layers[0].mix, model.layers[1].mix, model.layers[2].mix
    o = gru.qfv.offsets
    assert torch.equal(gru.qfv.weight[o["f"][0]:o["f"][0] + o["f"][1]], w["l0.mix.f"])
    assert torch.equal(gru.qfv.weight[o["v"][0]:], w["l0.mix.v"])
    assert torch.equal(gru.f_bias, w["l0.mix.f.b"]) and torch.equal(gru.lower, w["l0.mix.lower"])
    assert gru.norm.numel() == gru.Dv and torch.equal(gru.norm, w["l0.mix.norm"])
    H, D, C, Dv = lat.H, lat.D, lat.C, lat.Dv
    assert lat.R == 0 and not lat.gated and "g" not in lat.qcg.offsets
    assert torch.equal(lat.uk_t[1], w["l1.mix.uk"][D:2 * D].T) and lat.uk_t.shape == (H, C, D)
    assert torch.equal(lat.uv[2], w["l1.mix.uv"][2 * Dv:3 * Dv]) and torch.equal(lat.c_norm, w["l1.mix.dkv.norm"])
    assert torch.equal(lat.uq, w["l1.mix.uq"]) and torch.equal(lat.q_norm, w["l1.mix.dq.norm"]) and torch.equal(lat.sink, w["l1.mix.sink"])
    o = lat.qcg.offsets
    assert torch.equal(lat.qcg.weight[o["dq"][0]:o["dq"][0] + o["dq"][1]], w["l1.mix.dq"])
    assert torch.equal(lat.qcg.weight[o["dkv"][0]:o["dkv"][0] + o["dkv"][1]], w["l1.mix.dkv"])
    o = lin.qkvg.offsets
    assert torch.equal(lin.qkvg.weight[o["k"][0]:o["k"][0] + o["k"][1]], w["l2.mix.k"])
    assert torch.equal(lin.qkvg.weight[o["g"][0]:], w["l2.mix.g"]) and lin.norm.numel() == lin.H * lin.Dv
    assert torch.allclose(lin.decay.double(), torch.tensor(MIXED["layers"][2]["mixer"]["decay"]).double(), atol=1e-7)
    L0 = model.layers[0]
    assert torch.equal(L0.conv.weight, w["l0.canon1"]) and torch.equal(L0.out1.gate, w["l0.rg1"])
    assert torch.equal(L0.out1.gate_b, w["l0.rg1.b"]) and torch.equal(L0.out1.weight, w["l0.norm1b"])
    assert torch.equal(L0.out2.gate_b, w["l0.rg2.b"]) and torch.equal(L0.out2.weight, w["l0.norm2b"])
    assert torch.equal(L0.mlp.up[4], w["l0.mlp.e4.up"]) and torch.equal(L0.mlp.correction, w["l0.mlp.correction"])
    assert (L0.mlp.groups, L0.mlp.keep, L0.mlp.top_k) == (4, 2, 3) and L0.mlp.n_out == L0.mlp.E == 12
    assert model.layers[2].mlp is None and model.layers[2].norm2 is None and model.layers[2].out2 is None
    assert torch.equal(model.embed, w["embed"]) and not hasattr(model, "head")
    assert set(w) == set(F.tensor_shapes(MIXED))


def test_pages_and_state_of_a_sequence(model_dir):
    from nanovllm.models.felolorn import FelolornConfig, FelolornForCausalLM

    model = FelolornForCausalLM(FelolornConfig.from_dir(model_dir))
    # pages: the key/value latent of the latent layers only - not heads * (dim + vdim)
    assert model.cache_bytes_per_block(16, 2) == 16 * (40 + 64) * 2
    # a slot: taps - 1 rows of every layer's convolution input, plus the linear layers' matrix states, which the kernel
    # keeps padded: key channels to 64, value channels to a multiple of 32
    conv = 6 * 2 * MIXED["width"]
    states = 2 * 64 * 64 + 3 * 64 * 32 + 2 * 64 * 32 + 5 * 64 * 32
    assert model.state_bytes_per_slot() == 4 * (conv + states)
    only_latent = FelolornForCausalLM(FelolornConfig(config([with_mlp(latent(), None)], taps=1)))
    assert only_latent.state_bytes_per_slot() == 4 * 80          # (a one-tap convolution keeps a dummy row)
    only_recurrent = FelolornForCausalLM(FelolornConfig(config([with_mlp(hgrn2(), None)])))
    assert only_recurrent.cache_bytes_per_block(16, 2) == 0


def test_synthetic_checkpoint_names_match_the_design(model_dir):
    from nanovllm.models.felolorn import FelolornConfig, FelolornForCausalLM

    model = FelolornForCausalLM(FelolornConfig.from_dir(model_dir))
    got = {name: tuple(t.shape) for name, t in model.synthetic_state(0)}
    assert got == {k: tuple(v) for k, v in F.tensor_shapes(MIXED).items()}


def test_unknown_parts_are_refused():
    from nanovllm.models.felolorn import FelolornConfig, FelolornForCausalLM

    with pytest.raises(NotImplementedError):
        FelolornForCausalLM(FelolornConfig(config([{"type": "convolution", "mixer": {"heads": 1, "dim": 1, "vdim": 1}, "mlp": None}])))
    with pytest.raises(NotImplementedError):
        FelolornForCausalLM(FelolornConfig(config([with_mlp(lightning(), {"kind": "dense", "ff": 8})])))


# ---- the plain statement against itself -------------------------------------------------------------------------------
def test_plain_model_is_causal():
    cfg = config([with_mlp(lightning(), None), with_mlp(latent(), moe()), with_mlp(hgrn2(), None)], width=48, vocab=31, taps=4)
    w = F.random_model(cfg, seed=2)
    toks = list(range(30))
    full = F.forward(cfg, w, toks)
    assert torch.allclose(F.forward(cfg, w, toks[:17]), full[:17], atol=1e-10)


def test_plain_linear_attentions_equal_their_unrolled_sums():
    """o_t = sum_{s <= t} (prod of the decays after s) (q_t . k_s) v_s, written out without a state."""
    torch.manual_seed(0)
    T, W, H, D, Dv = 7, 10, 2, 3, 4
    u = torch.randn(T, W).double()
    p = {k: torch.randn(*s).double() for k, s in {"q": (H * D, W), "k": (H * D, W), "v": (H * Dv, W), "g": (H * Dv, W),
                                                   "norm": (H * Dv,), "o": (W, H * Dv), "f": (H * D, W), "f.b": (H * D,)}.items()}
    p["lower"] = torch.rand(H * D).double()
    m = {"heads": H, "dim": D, "vdim": Dv, "decay": [0.9, 0.5]}
    q, k, v = F.silu(u @ p["q"].T).view(T, H, D), F.silu(u @ p["k"].T).view(T, H, D), F.silu(u @ p["v"].T).view(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            for h in range(H):
                o[t, h] += m["decay"][h] ** (t - s) * (q[t, h] @ k[s, h]) * v[s, h]
    want = (F.rms_norm(o.reshape(T, H * Dv), p["norm"], 1e-6) * torch.sigmoid(u @ p["g"].T)) @ p["o"].T
    assert torch.allclose(F.lightning_mixer(u, p, m, 1e-6), want, atol=1e-10)
    p2 = dict(p, norm=torch.randn(Dv).double())
    f = (p["lower"] + (1 - p["lower"]) * torch.sigmoid(u @ p["f"].T + p["f.b"])).view(T, H, D)
    vv = (u @ p["v"].T).view(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            fade = torch.ones(H, D, dtype=torch.float64)
            for r in range(s + 1, t + 1):
                fade = fade * f[r]
            for h in range(H):
                o[t, h] += (q[t, h] * fade[h] * (1 - f[s, h])).sum() * vv[s, h]
    want = F.rms_norm(o, p2["norm"], 1e-6).reshape(T, H * Dv) @ p["o"].T
    assert torch.allclose(F.hgrn2_mixer(u, p2, m, 1e-6), want, atol=1e-10)


def test_plain_router_keeps_to_the_best_groups():
    """Choice scores all negative: experts of a dropped group must not come back through a zero."""
    z = torch.tensor([[3.0, 2.5, -4.0, -4.0, 2.9, -5.0]]).double()          # groups {0,1,2} {3,4,5}
    corr = torch.full((6,), -2.0).double()
    idx, wts = F.route(z, {"router": torch.eye(6).double(), "correction": corr},
                       {"experts": 6, "top": 3, "groups": {"count": 2, "keep": 1}})
    assert sorted(idx[0].tolist()) == [0, 1, 2]                               # 4 has the third-best score but sits outside
    assert torch.allclose(wts[0].sort().values, torch.sigmoid(z[0, :3]).sort().values)

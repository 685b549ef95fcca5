"""Host-side pieces of the Sanevik integration (no GPU): the configuration reader and the order of layer runs, the
checkpoint name map through the framework's loader, what a sequence needs in pages and state slots, the frequency table
of the rotations, and the plain statement's own consistency."""
import math
import os

import pytest
import torch

from oracle import sanevik as S
from sanevik_harness import LONG, MIXED, attention, config, moe, parallel, rot, with_mlp, write_model_dir


@pytest.fixture(scope="module")
def model_dir():
    return write_model_dir(MIXED, S.random_model(MIXED, seed=1))


def test_config_is_read_from_the_directory(model_dir):
    from nanovllm.config import Config

    c = Config(model_dir, dtype="float32", max_model_len=128, max_num_batched_tokens=128)
    hf = c.hf_config
    assert c.hybrid_state and hf.architectures == ["Sanevik"]
    assert (hf.vocab_size, hf.hidden_size, hf.num_hidden_layers) == (MIXED["vocab"], MIXED["width"], 5)
    assert (hf.loop_start, hf.loop_stop, hf.loop_times) == (1, 4, 3) and hf.norm_eps == 1e-5
    assert c.eos == -1 and c.max_model_len == 128


def test_order_of_layer_runs():
    """(layer, lane, number of the pass that begins here) in execution order, for a loop over a prefix, the middle, the
    tail, everything, nothing, and no loop at all; the same order as the plain statement's."""
    from nanovllm.models.sanevik import SanevikConfig

    layers = [with_mlp(attention(), None)] * 4
    for loop in ((0, 2, 2), (1, 3, 3), (2, 4, 2), (0, 4, 2), (0, 4, 1), (2, 2, 5), (0, 0, 0)):
        cfg = config(layers, loop=loop)
        c = SanevikConfig(cfg)
        assert [(i, t) for i, _, t in c.layer_runs] == S.layer_runs(cfg), loop
        for i, lane, t in c.layer_runs:
            assert 0 <= lane < c.lanes_of(i) and (t is None or t == lane)
    c = SanevikConfig(config(layers, loop=(1, 3, 3)))
    assert c.layer_runs == [(0, 0, None), (1, 0, 0), (2, 0, None), (1, 1, 1), (2, 1, None), (1, 2, 2), (2, 2, None), (3, 0, None)]
    assert [c.lanes_of(i) for i in range(4)] == [1, 3, 3, 1]


def test_every_tensor_lands_in_a_parameter(model_dir):
    """Load through the framework's loader on the CPU: every parameter is written, merged and stacked ones in the right
    row / column ranges, and nothing of the checkpoint is left over."""
    from nanovllm.models.sanevik import SanevikConfig, SanevikForCausalLM
    from nanovllm.utils.loader import load_model
    from safetensors.torch import load_file

    model = SanevikForCausalLM(SanevikConfig.from_dir(model_dir))
    for p in model.parameters():
        p.data.fill_(float("nan"))
    load_model(model, model_dir)
    w = {k: v.float() for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    for name, p in model.named_parameters():
        assert not torch.isnan(p).any(), name
    assert sum(p.numel() for p in model.parameters()) == sum(v.numel() for v in w.values())
    par, att = model.layers[0].mix, model.layers[1].mix

    def rows(m, name):
        off, n = m.offsets[name]
        return m.weight[off:off + n]

    for n in ("q", "k", "v"):
        assert torch.equal(rows(par.proj, "left." + n), w["l0.mix.left." + n])
        assert torch.equal(rows(par.left.conv, n), w[f"l0.mix.left.{n}.conv"])
        assert torch.equal(rows(att.qkv, n), w["l1.mix." + n])
    for n in ("q", "k", "v", "g"):
        assert torch.equal(rows(par.proj, "right." + n), w["l0.mix.right." + n])
    nl = par.left.out_features
    assert torch.equal(par.o[:, :nl], w["l0.mix.left.o"]) and torch.equal(par.o[:, nl:], w["l0.mix.right.o"])
    assert torch.equal(par.left.talk, w["l0.mix.left.talk"]) and par.left.sink is None
    assert torch.equal(att.attn.sink, w["l1.mix.sink"]) and att.attn.talk is None and att.attn.conv is None
    assert torch.equal(att.o, w["l1.mix.o"])
    m0 = MIXED["layers"][0]["mixer"]
    assert torch.allclose(par.right.decay.double(), torch.tensor(m0["right"]["decay"]).double(), atol=1e-7)
    assert (par.left_scale, par.right_scale, par.left.softcap, par.left.window) == (0.7, 1.2, 3.0, 13)
    assert att.attn.unit_norm and not par.left.unit_norm and att.attn.window == 17 and att.attn.rot_amp > 1.0
    L0 = model.layers[0]
    assert torch.equal(L0.norm1, w["l0.norm1"]) and torch.equal(L0.norm2, w["l0.norm2"])
    assert torch.equal(L0.mlp.up[4], w["l0.mlp.e4.up"]) and torch.equal(L0.mlp.router, w["l0.mlp.router"])
    assert (L0.mlp.E, L0.mlp.top_k, L0.mlp.limit) == (7, 3, 1.0)
    assert model.layers[2].mlp is None and model.layers[2].norm2 is None
    assert torch.equal(model.embed, w["embed"]) and torch.equal(model.loop_step, w["loop.step"])
    assert torch.equal(model.final_norm, w["final.norm"])
    assert set(w) == set(S.tensor_shapes(MIXED))


def test_pages_and_state_of_a_sequence(model_dir):
    from nanovllm.models.sanevik import SanevikConfig, SanevikForCausalLM

    model = SanevikForCausalLM(SanevikConfig.from_dir(model_dir))
    # pages: K and V rows of every attention, three times for the layers inside the loop
    per_token = (2 * 16 + 2 * 24) + 3 * ((3 * 24 + 3 * 20) + (2 * 32 + 2 * 32) + (4 * 32 + 4 * 16)) + (10 + 6)
    assert model.cache_bytes_per_block(16, 2) == 16 * per_token * 2
    # a slot: the convolutions' taps - 1 projected rows and the retention's matrix state (the kernel keeps it padded: key
    # channels to 64, value channels to a multiple of 32), three times inside the loop
    conv0, conv2 = 2 * (4 * 16 + 2 * 16 + 2 * 24), 1 * (2 * 32 + 2 * 32 + 2 * 32)
    assert model.state_bytes_per_slot() == 4 * ((conv0 + 3 * 64 * 32) + 3 * (conv2 + 2 * 64 * 32))
    only_attention = SanevikForCausalLM(SanevikConfig(config([with_mlp(attention(), None)])))
    assert only_attention.state_bytes_per_slot() == 0
    shapes = model.layers[0].mix.left.cache_shapes(7, 16)
    assert shapes == ((7, 2, 16, 16), (7, 1, 16, 48))      # mixed heads' weights: the value heads side by side in one row
    assert model.layers[1].mix.attn.cache_shapes(7, 16) == ((7, 3, 16, 24), (7, 3, 16, 20))


def test_synthetic_checkpoint_names_match_the_design(model_dir):
    from nanovllm.models.sanevik import SanevikConfig, SanevikForCausalLM

    model = SanevikForCausalLM(SanevikConfig.from_dir(model_dir))
    got = {name: tuple(t.shape) for name, t in model.synthetic_state(0)}
    assert got == {k: tuple(v) for k, v in S.tensor_shapes(MIXED).items()}


def test_unknown_parts_are_refused():
    from nanovllm.models.sanevik import SanevikConfig, SanevikForCausalLM

    with pytest.raises(NotImplementedError):
        SanevikForCausalLM(SanevikConfig(config([{"type": "convolution", "mixer": {}, "mlp": None}])))
    with pytest.raises(NotImplementedError):
        SanevikForCausalLM(SanevikConfig(config([with_mlp(attention(), {"kind": "dense", "ff": 8})])))


def test_frequency_table():
    """The product's table (double on the host, rounded once) against the plain statement's, with and without the
    long-context ramp; the ramp's ends: fast pairs untouched, slow pairs divided by the factor."""
    from nanovllm.layers.seqmix import rotary_table

    for dims, base, sc in ((16, 10000.0, LONG), (24, 300.0, None), (64, 20000.0, {"factor": 4.0, "original": 1024, "fast": 16.0, "slow": 2.0}),
                           (2, 5.0, {"factor": 2.0, "original": 8, "fast": 1.0, "slow": 1.0})):
        f, amp = rotary_table(dims, base, sc)
        want, want_amp = S.rotary_frequencies(rot(dims, base, sc))
        assert torch.allclose(f.double(), torch.tensor(want).double(), rtol=1e-7) and abs(amp - want_amp) < 1e-12
    f, amp = rotary_table(64, 20000.0, {"factor": 4.0, "original": 1024, "fast": 16.0, "slow": 2.0})
    plain = [20000.0 ** (-2.0 * i / 64) for i in range(32)]
    assert abs(float(f[0]) - plain[0]) < 1e-7 and abs(float(f[31]) - plain[31] / 4.0) < 1e-9
    assert abs(amp - (0.1 * math.log(4.0) + 1.0)) < 1e-12


# ---- the plain statement against itself -------------------------------------------------------------------------------
def test_plain_model_is_causal():
    cfg = config([with_mlp(parallel(), moe()), with_mlp(attention(), None)], width=48, vocab=31, loop=(0, 2, 2))
    w = S.random_model(cfg, seed=2)
    toks = list(range(30))
    full = S.forward(cfg, w, toks)
    assert torch.allclose(S.forward(cfg, w, toks[:17]), full[:17], atol=1e-10)


def test_plain_rotations_turn_pairs_by_the_position():
    """Scores of rotated queries and keys depend on the distance only; both pairings turn the same planes up to a
    permutation of the channels; channels beyond the rotated part pass through."""
    torch.manual_seed(0)
    r = rot(6, 100.0)
    x = torch.randn(1, 1, 8).double().expand(9, 1, 8)
    y = torch.randn(1, 1, 8).double().expand(9, 1, 8)
    for layout in ("interleaved", "halves"):
        a, b = S.rotate(x, r, layout), S.rotate(y, r, layout)
        d = (a[5, 0] * b[2, 0]).sum()
        assert torch.allclose((a[8, 0] * b[5, 0]).sum(), d, atol=1e-12)
        assert torch.equal(a[:, :, 6:], x[:, :, 6:])
    perm = [0, 2, 4, 1, 3, 5, 6, 7]            # halves layout of an interleaved vector
    inter = S.rotate(x, r, "interleaved")
    halves = S.rotate(x[:, :, perm], r, "halves")
    assert torch.allclose(inter[:, :, perm], halves, atol=1e-12)


def test_plain_retention_equals_its_unrolled_sum():
    """o_t = sum_{s <= t} decay^(t - s) (q_t . k_s) v_s, written out without a state."""
    torch.manual_seed(0)
    T, W, H, D, Dv = 7, 10, 2, 4, 3
    h = torch.randn(T, W).double()
    p = {k: torch.randn(*s).double() for k, s in {"q": (H * D, W), "k": (H * D, W), "v": (H * Dv, W), "g": (H * Dv, W),
                                                   "o": (W, H * Dv)}.items()}
    m = {"heads": H, "dim": D, "vdim": Dv, "decay": [0.9, 0.5], "rot": rot(4, 50.0)}
    q = S.rotate((h @ p["q"].T).view(T, H, D), m["rot"], "halves")
    k = S.rotate((h @ p["k"].T).view(T, H, D), m["rot"], "halves") * D ** -0.5
    v = (h @ p["v"].T).view(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            for hd in range(H):
                o[t, hd] += m["decay"][hd] ** (t - s) * (q[t, hd] @ k[s, hd]) * v[s, hd]
    want = (S.rms_unit(o, 1e-6).reshape(T, H * Dv) * S.silu(h @ p["g"].T)) @ p["o"].T
    assert torch.allclose(S.retention_mixer(h, p, m, 1e-6), want, atol=1e-10)


def test_plain_experts_take_their_weight_on_the_input():
    """With a limit that bites, expert(s h) is not s expert(h); the chosen experts are those of the largest scores."""
    torch.manual_seed(1)
    W, F, E = 6, 5, 4
    p = {"router": torch.randn(E, W).double()}
    for e in range(E):
        p.update({f"e{e}.gate": torch.randn(F, W).double() * 3, f"e{e}.up": torch.randn(F, W).double() * 3,
                  f"e{e}.down": torch.randn(W, F).double()})
    ml = moe(ff=F, experts=E, top=2, limit=0.5)
    h = torch.randn(3, W).double()
    out = S.sparse_ff(h, p, ml)
    s = torch.sigmoid(h @ p["router"].T)
    for t in range(3):
        best = s[t].argsort(descending=True)[:2]
        inside = sum(S.expert_ff(s[t, e] * h[t:t + 1], p, int(e), 0.5)[0] for e in best)
        outside = sum(s[t, e] * S.expert_ff(h[t:t + 1], p, int(e), 0.5)[0] for e in best)
        assert torch.allclose(out[t], inside, atol=1e-12) and not torch.allclose(inside, outside, atol=1e-3)

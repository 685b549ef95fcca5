"""Felolorn: a decoder whose layers - in an order its configuration lists - mix the sequence with a latent attention
that knows no positions (queries through a latent of their own, a sink logit per head in the softmax), a linear
attention whose state fades by a constant per head, or a linear attention whose forget gate also writes; each followed
by a group-routed sparse feed-forward (or none).  Every sublayer sits between two RMS norms, reads - the mixers - its
input through a short causal convolution beside the identity, and reaches the fp32 residual stream through a sigmoid
gate computed from its own input:

    h = n(x; w_1);  x <- x + n(sigmoid(W_rg1 h + b) * mixer(h + conv(h)); w_1b)
    h = n(x; w_2);  x <- x + n(sigmoid(W_rg2 h + b) * ff(h); w_2b)

The mechanisms are the classes of layers/seqmix.py; this file reads the configuration, wires the layers, names the
checkpoint's tensors and says what cache and state a sequence needs:

  config.json   {"architecture": "Felolorn", "vocab", "width", "norm": {"eps"}, "canon": {"taps"}, "embedding": {"scale"},
                "logit_softcap", "layers": [{"type": "latent_attention" | "lightning" | "hgrn2", "mixer": {...},
                "mlp": {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top", "groups": {"count", "keep"}}} | null}]}
  checkpoint    embed (also the output projection), final.norm, l<i>.norm1 / norm1b / norm2 / norm2b, l<i>.canon1,
                l<i>.rg1(.b) / rg2(.b), l<i>.mix.<name>, l<i>.mlp.<name>
  per sequence  pages: one latent row per token and latent-attention layer; a state slot: the convolution's last
                taps - 1 inputs of EVERY layer and the fp32 matrix state of every linear-attention layer
"""
from __future__ import annotations

import json
import os

import torch
from torch import nn

from nanovllm import _C, ops
from nanovllm.layers.seqmix import (ForgetGateLinearAttention, GatedOutputNorm, GroupedSparseMLP, HeadDecayLinearAttention,
                                    InputConvolution, LatentAttention, _vector)


class FelolornConfig:
    """config.json of this design with the attribute names the engine reads from a configuration object."""
    architectures = ["Felolorn"]
    model_type = "felolorn"
    max_position_embeddings = None   # nothing in the design depends on absolute positions
    eos_token_id = None
    native = True                    # not a transformers configuration

    def __init__(self, raw: dict, dtype: str = "bfloat16"):
        self.raw = raw
        self.vocab_size, self.hidden_size = int(raw["vocab"]), int(raw["width"])
        self.layers = raw["layers"]
        self.num_hidden_layers = len(self.layers)
        self.norm_eps = float(raw["norm"]["eps"])
        self.conv_taps = int(raw["canon"]["taps"])
        self.embedding_scale = float((raw.get("embedding") or {}).get("scale", 1.0))
        self.logit_softcap = float(raw.get("logit_softcap") or 0.0)   # 0: logits are not capped
        self.torch_dtype = dtype

    @classmethod
    def from_dir(cls, path: str, dtype: str = "bfloat16") -> "FelolornConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls(json.load(f), dtype)


class FelolornLayer(nn.Module):
    def __init__(self, cfg: FelolornConfig, index: int):
        super().__init__()
        spec, W, eps = cfg.layers[index], cfg.hidden_size, cfg.norm_eps
        m = spec["mixer"]
        self.kind = spec["type"]
        H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        if self.kind == "latent_attention":
            self.mix = LatentAttention(W, H, D, 0, Dv, int(m["kv_rank"]), 0, 1.0, float(m["scale"]), eps,
                                       q_rank=int(m["q_rank"]), gate=False, sink=True)
        elif self.kind == "lightning":
            decay = m["decay"]
            self.mix = HeadDecayLinearAttention(W, H, D, Dv, decay if isinstance(decay, (list, tuple)) else [decay] * H, eps)
        elif self.kind == "hgrn2":
            self.mix = ForgetGateLinearAttention(W, H, D, Dv, eps)
        else:
            raise NotImplementedError(f"layer {index}: mixer type {self.kind!r}")
        self.norm1 = _vector(W, 1.0)
        self.conv = InputConvolution(W, cfg.conv_taps)
        self.out1 = GatedOutputNorm(W, eps)
        ml = spec.get("mlp")
        self.mlp = self.norm2 = self.out2 = None
        if ml is not None:
            if ml.get("kind", "moe") != "moe":
                raise NotImplementedError(f"layer {index}: feed-forward kind {ml.get('kind')!r}")
            r = ml["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            self.mlp = GroupedSparseMLP(W, int(ml["expert"]["ff"]), int(r["experts"]), 0, int(r["top"]), int(g["count"]),
                                        int(g["keep"]), score="sigmoid", group_value="top2")
            self.norm2 = _vector(W, 1.0)
            self.out2 = GatedOutputNorm(W, eps)


class FelolornForCausalLM(nn.Module):
    hybrid_state = True   # sequences own state slots beside their pages: ModelRunner takes the row-step path
    fp32_residual = True

    def __init__(self, config: FelolornConfig):
        super().__init__()
        self.config = config
        W, V = config.hidden_size, config.vocab_size
        self.embed = nn.Parameter(torch.empty(V, W), requires_grad=False)   # input table and output projection
        self.layers = nn.ModuleList([FelolornLayer(config, i) for i in range(len(config.layers))])
        self.final_norm = _vector(W, 1.0)
        self.trace_layers: list | None = None  # bring-up hook: receives a copy of the residual stream after every layer

    # ---- checkpoint names -> parameters (utils/loader.py) ------------------------------------------------------
    def map_checkpoint_name(self, name: str):
        """-> parameter path, (parameter path, shard) for tensors that land inside a merged / stacked parameter, or None
        for a tensor this configuration has no use for."""
        if name == "embed":
            return name
        if name == "final.norm":
            return "final_norm"
        layer, rest = name.split(".", 1)
        i = int(layer[1:])
        pre, L = f"layers.{i}.", self.layers[i]
        if rest == "norm1":
            return pre + "norm1"
        if rest == "canon1":
            return pre + "conv.weight"
        second = {"norm2": "norm2", "norm2b": "out2.weight", "rg2": "out2.gate", "rg2.b": "out2.gate_b"}
        if rest in second:
            return pre + second[rest] if L.mlp is not None else None
        first = {"norm1b": "out1.weight", "rg1": "out1.gate", "rg1.b": "out1.gate_b"}
        if rest in first:
            return pre + first[rest]
        part, leaf = rest.split(".", 1)
        if part == "mlp":
            if leaf in ("router", "correction"):
                return pre + "mlp." + leaf
            expert, proj = leaf.split(".")
            return pre + "mlp." + proj, int(expert[1:])
        if L.kind == "latent_attention":
            if leaf in ("dq", "dkv"):
                return pre + "mix.qcg.weight", leaf
            return pre + "mix." + {"dq.norm": "q_norm", "uq": "uq", "dkv.norm": "c_norm", "uk": "uk_t", "uv": "uv",
                                   "sink": "sink", "o": "o"}[leaf]
        if L.kind == "lightning":
            if leaf in ("q", "k", "v", "g"):
                return pre + "mix.qkvg.weight", leaf
            return pre + "mix." + leaf  # norm, o
        if leaf in ("q", "f", "v"):
            return pre + "mix.qfv.weight", leaf
        return pre + "mix." + {"f.b": "f_bias", "lower": "lower", "norm": "norm", "o": "o"}[leaf]

    def synthetic_state(self, seed: int = 0):
        """Random tensors under the checkpoint's names (no-checkpoint mode: benchmarks)."""
        g = torch.Generator().manual_seed(seed)
        cfg, W = self.config, self.config.hidden_size

        def mat(*shape, std=None):
            return torch.randn(*shape, generator=g) * (std if std is not None else shape[-1] ** -0.5)

        yield "embed", mat(cfg.vocab_size, W, std=W ** -0.5)
        yield "final.norm", 1 + mat(W, std=0.05)
        for i, layer in enumerate(self.layers):
            mx, p = layer.mix, f"l{i}."
            yield p + "norm1", 1 + mat(W, std=0.05)
            yield p + "norm1b", 1 + mat(W, std=0.05)
            yield p + "canon1", mat(W, cfg.conv_taps, std=0.3)
            yield p + "rg1", mat(W, W)
            yield p + "rg1.b", mat(W, std=0.3)
            if layer.kind == "latent_attention":
                yield p + "mix.dq", mat(mx.Q, W)
                yield p + "mix.dq.norm", 1 + mat(mx.Q, std=0.05)
                yield p + "mix.uq", mat(mx.H * mx.D, mx.Q)
                yield p + "mix.dkv", mat(mx.C, W)
                yield p + "mix.dkv.norm", 1 + mat(mx.C, std=0.05)
                yield p + "mix.uk", mat(mx.H * mx.D, mx.C)
                yield p + "mix.uv", mat(mx.H * mx.Dv, mx.C)
                yield p + "mix.sink", mat(mx.H, std=1.0)
            elif layer.kind == "lightning":
                for n, (_, rows) in mx.qkvg.offsets.items():
                    yield p + "mix." + n, mat(rows, W)
                yield p + "mix.norm", 1 + mat(mx.H * mx.Dv, std=0.05)
            else:
                for n, (_, rows) in mx.qfv.offsets.items():
                    yield p + "mix." + n, mat(rows, W)
                yield p + "mix.f.b", mat(mx.H * mx.D, std=0.5)
                yield p + "mix.lower", torch.rand(mx.H * mx.D, generator=g) * 0.9
                yield p + "mix.norm", 1 + mat(mx.Dv, std=0.05)
            yield p + "mix.o", mat(W, mx.H * mx.Dv)
            ml = layer.mlp
            if ml is None:
                continue
            yield p + "norm2", 1 + mat(W, std=0.05)
            yield p + "norm2b", 1 + mat(W, std=0.05)
            yield p + "rg2", mat(W, W)
            yield p + "rg2.b", mat(W, std=0.3)
            yield p + "mlp.router", mat(ml.n_out, W)
            yield p + "mlp.correction", mat(ml.n_out, std=0.1)
            ff = ml.gate.shape[1]
            for e in range(ml.E):
                yield p + f"mlp.e{e}.gate", mat(ff, W)
                yield p + f"mlp.e{e}.up", mat(ff, W)
                yield p + f"mlp.e{e}.down", mat(W, ff)

    # ---- cache and state ------------------------------------------------------------------------------------------
    def cache_bytes_per_block(self, block_size: int, itemsize: int) -> int:
        return block_size * itemsize * sum(l.mix.C + l.mix.R for l in self.layers if l.kind == "latent_attention")

    def state_bytes_per_slot(self) -> int:
        n = 0
        for l in self.layers:
            c = l.conv.state_shape(1)
            n += c[1] * c[2]
            if l.kind != "latent_attention":
                n += l.mix.state_shape(1)[1]
        return 4 * n

    def bind_cache(self, num_blocks: int, block_size: int, n_slots: int, dtype: torch.dtype, device) -> None:
        """Pages for the latent rows (serving dtype), state slots for the convolutions' tails and the matrix states
        (fp32).  Nothing has to be cleared when a page or a slot changes hands: a sequence's first row starts every state
        from zero and no kernel reads a cache row its own sequence has not written."""
        for l in self.layers:
            l.conv.state = torch.zeros(l.conv.state_shape(n_slots), dtype=torch.float32, device=device)
            if l.kind == "latent_attention":
                l.mix.cache = torch.zeros(l.mix.cache_shape(num_blocks, block_size), dtype=dtype, device=device)
            else:
                l.mix.state = torch.zeros(l.mix.state_shape(n_slots), dtype=torch.float32, device=device)

    # ---- one step over the rows the context describes ----------------------------------------------------------------
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor | None = None) -> torch.Tensor:
        cfg, n = self.config, len(self.layers)
        x = ops.embedding_f32(input_ids, self.embed, scale=cfg.embedding_scale)
        h = ops.add_rmsnorm_f32(x, None, 0.0, self.layers[0].norm1, cfg.norm_eps)
        for i, layer in enumerate(self.layers):
            after = self.layers[i + 1].norm1 if i + 1 < n else None   # (the output's norm is taken of the wanted rows only)
            gate = layer.out1.gate_of(h)
            y = layer.mix(layer.conv(h))
            h = layer.out1.add_to(x, y, gate, layer.norm2 if layer.mlp is not None else after)
            if layer.mlp is not None:
                gate = layer.out2.gate_of(h)
                h = layer.out2.add_to(x, layer.mlp(h), gate, after)
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        return x

    def compute_logits(self, hidden: torch.Tensor, rows: torch.Tensor | None = None) -> torch.Tensor:
        """fp32 logits of the given rows (default: all): the table itself is the projection; cap * tanh(z / cap)."""
        if rows is not None:
            hidden = hidden.index_select(0, rows)
        h = ops.add_rmsnorm_f32(hidden, None, 0.0, self.final_norm, self.config.norm_eps)
        cap = self.config.logit_softcap
        if cap > 0:
            return ops.gemm_any_act(h, self.embed, act=_C.ACT_SOFTCAP, alpha=cap)
        return ops.gemm_any(h, self.embed)

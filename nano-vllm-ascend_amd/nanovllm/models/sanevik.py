"""Sanevik: a pre-norm decoder (x <- x + mixer(n(x)), x <- x + ff(n(x)), n(x; w) = x / sqrt(mean x^2 + eps) (1 + w), fp32
residual) whose configuration lists its layers and may run a stretch of them several times with the same weights:

  order        layers [0, start), then `times` passes over [start, stop), then [stop, n).  Pass t begins with
               x <- x + step[t] (+ the embedding rows from the second pass on).  Every pass has K/V pages and recurrent
               state of its own: a looped layer keeps one cache / state per pass ("lane").
  attention    sliding-window attention over rotated (interleaved pairs, long-context frequency ramp), then unit-normed
               query and key heads, a sink logit per head in the softmax
  parallel     two mixers on the same input, summed with fixed scales: a sliding-window attention behind short causal
               convolutions with capped scores and mixing of the heads' softmax weights, and a retention (linear attention,
               fixed decay per head, rotated in half-split pairs) with unit-normed heads and a SiLU gate
  feed-forward top-k experts by sigmoid score, the score multiplying the expert's input; capped / clamped gated experts

The mechanisms are the classes of layers/seqmix.py; this file reads the configuration, wires the layers, names the
checkpoint's tensors and says what cache and state a sequence needs:

  config.json   {"architecture": "Sanevik", "vocab", "width", "norm": {"eps"}, "loop": {"start", "stop", "times"} | absent,
                "layers": [{"type": "attention" | "parallel", "mixer": {...}, "mlp": {"kind": "moe", "expert": {"ff",
                "limit"}, "router": {"experts", "top"}} | null}]}
  checkpoint    embed (also the output projection), final.norm, loop.step, l<i>.norm1 / norm2, l<i>.mix.<name>
                (parallel: l<i>.mix.left.<name>, l<i>.mix.right.<name>), l<i>.mlp.router, l<i>.mlp.e<k>.gate / up / down
  per sequence  pages: K / V rows of every attention, once per pass; a state slot: the convolutions' last taps - 1
                projected rows and the retention's fp32 matrix state, once per pass
"""
from __future__ import annotations

import json
import os

import torch
from torch import nn

from nanovllm import ops
from nanovllm.layers.seqmix import (CAUSAL, InputWeightedSparseMLP, ParallelMixers, Retention, RotaryWindowAttention,
                                    SinkAttentionMixer, _vector)


class SanevikConfig:
    """config.json of this design with the attribute names the engine reads from a configuration object."""
    architectures = ["Sanevik"]
    model_type = "sanevik"
    max_position_embeddings = None
    eos_token_id = None
    native = True                    # not a transformers configuration

    def __init__(self, raw: dict, dtype: str = "bfloat16"):
        self.raw = raw
        self.vocab_size, self.hidden_size = int(raw["vocab"]), int(raw["width"])
        self.layers = raw["layers"]
        self.num_hidden_layers = len(self.layers)
        self.norm_eps = float(raw["norm"]["eps"])
        loop = raw.get("loop")
        n = len(self.layers)
        self.loop_start, self.loop_stop, self.loop_times = (int(loop["start"]), int(loop["stop"]), int(loop["times"])) \
            if loop else (0, 0, 0)
        assert 0 <= self.loop_start <= self.loop_stop <= n and (not loop or self.loop_times >= 1), loop
        self.torch_dtype = dtype

    @property
    def layer_runs(self):
        """[(layer, lane, pass number on a pass's first layer or None)] in execution order"""
        a, b, n = self.loop_start, self.loop_stop, len(self.layers)
        if not self.loop_times or a == b:
            return [(i, 0, None) for i in range(n)]
        runs = [(i, 0, None) for i in range(a)]
        for t in range(self.loop_times):
            runs += [(i, t, t if i == a else None) for i in range(a, b)]
        return runs + [(i, 0, None) for i in range(b, n)]

    def lanes_of(self, i: int) -> int:
        return self.loop_times if self.loop_times and self.loop_start <= i < self.loop_stop else 1

    @classmethod
    def from_dir(cls, path: str, dtype: str = "bfloat16") -> "SanevikConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls(json.load(f), dtype)


def _window_attention(m: dict, eps: float, *, unit_norm: bool, sink: bool, talk: bool) -> RotaryWindowAttention:
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    return RotaryWindowAttention(int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]),
                                 int(m["mask"]["size"]) if m.get("mask") else CAUSAL, float(m["scale"]), eps,
                                 int(rot["dims"]), float(rot["base"]), rot.get("scaling"), unit_norm=unit_norm, sink=sink,
                                 softcap=float(m.get("softcap") or 0.0), conv_taps=int(m.get("conv") or 0), talk=talk)


class SanevikLayer(nn.Module):
    def __init__(self, cfg: SanevikConfig, index: int):
        super().__init__()
        spec, W, eps = cfg.layers[index], cfg.hidden_size, cfg.norm_eps
        m = spec["mixer"]
        self.kind, self.lanes = spec["type"], cfg.lanes_of(index)
        if self.kind == "attention":
            self.mix = SinkAttentionMixer(W, _window_attention(m, eps, unit_norm=True, sink=True, talk=False))
        elif self.kind == "parallel":
            r = m["right"]
            rot = r.get("rot") or {"dims": 0, "base": 1.0}
            right = Retention(int(r["heads"]), int(r["dim"]), int(r["vdim"]), r["decay"], eps, int(rot["dims"]),
                              float(rot["base"]), rot.get("scaling"))
            self.mix = ParallelMixers(W, _window_attention(m["left"], eps, unit_norm=False, sink=False, talk=True), right,
                                      float(m["left_scale"]), float(m["right_scale"]))
        else:
            raise NotImplementedError(f"layer {index}: mixer type {self.kind!r}")
        self.norm1 = _vector(W)
        ml = spec.get("mlp")
        self.mlp = self.norm2 = None
        if ml is not None:
            if ml.get("kind", "moe") != "moe":
                raise NotImplementedError(f"layer {index}: feed-forward kind {ml.get('kind')!r}")
            self.mlp = InputWeightedSparseMLP(W, int(ml["expert"]["ff"]), int(ml["router"]["experts"]),
                                              int(ml["router"]["top"]), float(ml["expert"]["limit"]))
            self.norm2 = _vector(W)

    @property
    def attention(self) -> RotaryWindowAttention:
        return self.mix.attn if self.kind == "attention" else self.mix.left


class SanevikForCausalLM(nn.Module):
    hybrid_state = True   # sequences own state slots beside their pages: ModelRunner takes the row-step path
    fp32_residual = True

    def __init__(self, config: SanevikConfig):
        super().__init__()
        self.config = config
        W, V = config.hidden_size, config.vocab_size
        self.embed = nn.Parameter(torch.empty(V, W), requires_grad=False)   # input table and output projection
        self.layers = nn.ModuleList([SanevikLayer(config, i) for i in range(len(config.layers))])
        self.final_norm = _vector(W)
        self.loop_step = nn.Parameter(torch.zeros(max(config.loop_times, 1), W, dtype=torch.float32), requires_grad=False)
        self.trace_layers: list | None = None  # bring-up hook: receives a copy of the residual stream after every layer run

    # ---- checkpoint names -> parameters (utils/loader.py) ------------------------------------------------------
    def map_checkpoint_name(self, name: str):
        """-> parameter path, (parameter path, shard) for tensors that land inside a merged / stacked parameter, or None
        for a tensor this configuration has no use for."""
        if name == "embed":
            return name
        if name == "final.norm":
            return "final_norm"
        if name == "loop.step":
            return "loop_step" if self.config.loop_times else None
        layer, rest = name.split(".", 1)
        i = int(layer[1:])
        pre, L = f"layers.{i}.", self.layers[i]
        if rest == "norm1":
            return pre + "norm1"
        if rest == "norm2":
            return pre + "norm2" if L.mlp is not None else None
        part, leaf = rest.split(".", 1)
        if part == "mlp":
            if leaf == "router":
                return pre + "mlp.router"
            expert, proj = leaf.split(".")
            return pre + "mlp." + proj, int(expert[1:])
        if L.kind == "attention":
            if leaf in ("q", "k", "v"):
                return pre + "mix.qkv.weight", leaf
            return pre + {"sink": "mix.attn.sink", "o": "mix.o"}[leaf]
        side, leaf = leaf.split(".", 1)
        if leaf == "o":
            return pre + "mix.o", side
        if side == "left":
            if leaf == "talk":
                return pre + "mix.left.talk"
            if leaf.endswith(".conv"):
                return (pre + "mix.left.conv.weight", leaf[:-5]) if L.mix.left.conv is not None else None
        return pre + "mix.proj.weight", f"{side}.{leaf}"

    def synthetic_state(self, seed: int = 0):
        """Random tensors under the checkpoint's names (no-checkpoint mode: benchmarks)."""
        g = torch.Generator().manual_seed(seed)
        cfg, W = self.config, self.config.hidden_size

        def mat(*shape, std=None):
            return torch.randn(*shape, generator=g) * (std if std is not None else shape[-1] ** -0.5)

        yield "embed", mat(cfg.vocab_size, W, std=W ** -0.5)
        yield "final.norm", mat(W, std=0.05)
        if cfg.loop_times:
            yield "loop.step", mat(cfg.loop_times, W, std=0.02)
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            yield p + "norm1", mat(W, std=0.05)
            if layer.kind == "attention":
                a = layer.mix.attn
                for n, rows in a.parts.items():
                    yield p + "mix." + n, mat(rows, W)
                yield p + "mix.sink", mat(a.H, std=1.0)
                yield p + "mix.o", mat(W, a.out_features)
            else:
                a, r = layer.mix.left, layer.mix.right
                for n, rows in a.parts.items():
                    yield p + "mix.left." + n, mat(rows, W)
                    if a.conv is not None:
                        yield p + f"mix.left.{n}.conv", mat(rows, a.conv.weight.shape[1], std=0.5)
                yield p + "mix.left.talk", torch.eye(a.H) + mat(a.H, a.H, std=0.2)
                yield p + "mix.left.o", mat(W, a.out_features)
                for n, rows in r.parts.items():
                    yield p + "mix.right." + n, mat(rows, W)
                yield p + "mix.right.o", mat(W, r.out_features)
            ml = layer.mlp
            if ml is None:
                continue
            yield p + "norm2", mat(W, std=0.05)
            yield p + "mlp.router", mat(ml.E, W)
            ff = ml.gate.shape[1]
            for e in range(ml.E):
                yield p + f"mlp.e{e}.gate", mat(ff, W)
                yield p + f"mlp.e{e}.up", mat(ff, W)
                yield p + f"mlp.e{e}.down", mat(W, ff)

    # ---- cache and state ------------------------------------------------------------------------------------------
    def cache_bytes_per_block(self, block_size: int, itemsize: int) -> int:
        n = 0
        for l in self.layers:
            a = l.attention
            n += l.lanes * (a.G * a.D + a.G * a.Dv)
        return block_size * itemsize * n

    def state_bytes_per_slot(self) -> int:
        n = 0
        for l in self.layers:
            if l.kind != "parallel":
                continue
            c = l.mix.left.conv_state_shape(1)
            n += l.lanes * ((c[1] * c[2] if c else 0) + l.mix.right.state_shape(1)[1])
        return 4 * n

    def bind_cache(self, num_blocks: int, block_size: int, n_slots: int, dtype: torch.dtype, device) -> None:
        """Pages for the K / V rows (serving dtype), state slots for the convolutions' tails and the retentions' matrix
        states (fp32), one set per pass of a looped layer.  Nothing has to be cleared when a page or a slot changes hands:
        a sequence's first row starts every state from zero and no kernel reads a cache row its own sequence has not
        written."""
        for l in self.layers:
            a = l.attention
            ks, vs = a.cache_shapes(num_blocks, block_size)
            a.k_cache = [torch.zeros(ks, dtype=dtype, device=device) for _ in range(l.lanes)]
            a.v_cache = [torch.zeros(vs, dtype=dtype, device=device) for _ in range(l.lanes)]
            if l.kind == "parallel":
                if a.conv is not None:
                    a.conv_state = [torch.zeros(a.conv_state_shape(n_slots), dtype=torch.float32, device=device)
                                    for _ in range(l.lanes)]
                r = l.mix.right
                r.state = [torch.zeros(r.state_shape(n_slots), dtype=torch.float32, device=device) for _ in range(l.lanes)]

    # ---- one step over the rows the context describes ----------------------------------------------------------------
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor | None = None) -> torch.Tensor:
        cfg = self.config
        eps, runs = cfg.norm_eps, cfg.layer_runs
        e = ops.embedding_f32(input_ids, self.embed)
        # (the embedding rows are needed again at the start of the later passes: the stream is a copy of its own then)
        x = e.clone() if cfg.loop_times > 1 and cfg.loop_stop > cfg.loop_start else e
        y = None   # the sublayer output that is still to be added to x
        for n, (i, lane, begins) in enumerate(runs):
            layer = self.layers[i]
            if begins is not None:
                # a pass begins: what the last layer left is added first (it belongs to that layer's result), then the
                # embedding rows (from the second pass on) and the pass's vector, with this layer's first norm
                if y is not None:
                    ops.add_rmsnorm_f32(x, y, 1.0, None, eps)
                h = ops.add_rmsnorm_f32(x, e if begins > 0 else None, 1.0, layer.norm1, eps, 1.0, vec=self.loop_step[begins])
            else:
                h = ops.add_rmsnorm_f32(x, y, 1.0, layer.norm1, eps, 1.0)
            y = layer.mix(h, lane)
            if layer.mlp is not None:
                y = layer.mlp(ops.add_rmsnorm_f32(x, y, 1.0, layer.norm2, eps, 1.0))
            if self.trace_layers is not None:
                ops.add_rmsnorm_f32(x, y, 1.0, None, eps)
                y = None
                self.trace_layers.append(x.clone())
        if y is not None:
            ops.add_rmsnorm_f32(x, y, 1.0, None, eps)
        return x

    def compute_logits(self, hidden: torch.Tensor, rows: torch.Tensor | None = None) -> torch.Tensor:
        """fp32 logits of the given rows (default: all): the embedding table itself is the projection."""
        if rows is not None:
            hidden = hidden.index_select(0, rows)
        h = ops.add_rmsnorm_f32(hidden, None, 0.0, self.final_norm, self.config.norm_eps, 1.0)
        return ops.gemm_any(h, self.embed)

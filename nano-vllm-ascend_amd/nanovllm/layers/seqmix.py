"""Layer classes of the 32-bit-residual model families (kernels: csrc/gemm_any.hip, csrc/seqmix.hip).

Each class is one mechanism with its constants as constructor arguments, so that a model file only wires them by its
configuration:

  OutputLayerNorm           LayerNorm (weight + bias) applied to a sublayer's OUTPUT and added to the residual
  SlidingWindowAttention    paged sliding-window attention, linear distance bias per head, whole-projection q / k RMS norm,
                            optional value mixing with an earlier layer's values, sigmoid output gate
  ChannelDeltaMixer         gated delta rule with a decay per head and key channel behind short causal convolutions;
                            recurrent state and convolution tail live in per-sequence state slots
  GroupedSparseMLP          sparse mixture of SwiGLU experts, group-limited top-k routing with a choice correction,
                            un-renormalised weights, identity experts
  DepthMixedResidual        pre-norm residual stream x <- x + m f(norm(x)) whose layers read a learned weighted sum of the
                            embedding and of all earlier layers' results; RMS norms with weights stored around zero
  MinGRUMixer               minimal gated recurrence (gates from the current token only), fp32 state per sequence slot
  LatentAttention           attention over a low-rank key/value latent plus one shared rotated key part; only those are
                            cached, the per-head up-projections are absorbed into the query and the output
  BiasedAttention           grouped-head causal attention with a log-distance bias per head and a position-dependent
                            query temperature, no rotation
  GatedDenseMLP             W_d (act(W_g h + b) * (W_u h + b)) + b
  SharedSparseMLP           top-k experts of the plain form W_d act(W_u h), softmax over the chosen logits, plus a shared
                            expert behind a per-token sigmoid gate
  InputConvolution          what a sublayer reads is h + conv(h): a short causal depthwise convolution beside the identity,
                            its last taps - 1 inputs carried in the sequence's state slot
  GatedOutputNorm           a sublayer's output times sigmoid(W h + b) of the sublayer's input, RMS-normed, added to the
                            residual; the same launch norms the sum for the next sublayer
  HeadDecayLinearAttention  linear attention with a matrix state per head that fades by one constant per head
  ForgetGateLinearAttention linear attention whose per-channel forget gate f also writes: S <- diag(f) S + (1 - f) v^T
  rotary_table              rotation frequencies of a head's channel pairs, optionally rescaled for long contexts (a ramp
                            between the fast pairs, kept, and the slow ones, divided by a factor; cos / sin amplified)
  RotaryWindowAttention     paged sliding-window attention over rotated (interleaved pairs) queries and keys, optionally
                            behind short causal convolutions, with unit-normed heads, a sink logit per head, capped scores
                            and mixing of the heads' softmax weights as options
  Retention                 linear attention over rotated (half-split pairs) queries and keys with a fixed decay per head,
                            per-head unit norm and a SiLU gate on the read-out
  SinkAttentionMixer        projections + RotaryWindowAttention + output projection
  ParallelMixers            a RotaryWindowAttention and a Retention side by side on the same input: one merged input
                            projection, one merged output projection of the two scaled read-outs
  InputWeightedSparseMLP    top-k experts by sigmoid score whose weight multiplies the expert's INPUT; experts
                            W_d (g sigmoid(1.702 g) (u + 1)) with g capped and u clamped

Layers whose weights a model runs several times per step (a looped stack) keep one cache / state per pass ("lane"): their
forward takes the lane's number.

Activations are fp32 tensors [rows, features]; matrices are stored in the serving dtype (bf16, or fp32 for the exact
mode), vectors always in fp32.  A step's rows come with the metadata of utils/context.py: cu_seqlens_q, kv_lens (the
sequences' lengths INCLUDING this step's rows), slot_mapping, block_tables, state_slots.  Prompt portions and single
decoded tokens are the same thing to every kernel here: a run of rows that continues a sequence.
"""
from __future__ import annotations

import torch
from torch import nn

from nanovllm import _C, ops
from nanovllm.utils.context import get_context


def _vector(n: int, fill: float = 0.0) -> nn.Parameter:
    return nn.Parameter(torch.full((n,), fill, dtype=torch.float32), requires_grad=False)


def _matrix(*shape) -> nn.Parameter:
    return nn.Parameter(torch.empty(*shape), requires_grad=False)  # (the default dtype = the serving dtype)


class MergedRows(nn.Module):
    """Several projections of the same input stacked along their output features (one GEMM instead of several); a
    checkpoint's separate tensors land in their row ranges through `weight_loader(param, tensor, shard_name)`."""

    def __init__(self, in_features: int, parts: dict[str, int], dtype=None, bias: bool = False):
        super().__init__()
        self.offsets, off = {}, 0
        for name, n in parts.items():
            self.offsets[name] = (off, n)
            off += n
        self.weight = nn.Parameter(torch.empty(off, in_features, dtype=dtype), requires_grad=False)
        self.weight.weight_loader = self._load
        self.bias = None
        if bias:  # fp32, zero where a part has none; loaded by row range like the weight
            self.bias = _vector(off)
            self.bias.weight_loader = self._load

    def _load(self, param, tensor, shard):
        off, n = self.offsets[shard]
        assert tensor.shape[0] == n, (shard, tuple(tensor.shape), n)
        param.data[off:off + n].copy_(tensor)

    def cols(self, y: torch.Tensor, name: str) -> torch.Tensor:
        off, n = self.offsets[name]
        return y[:, off:off + n]

    def forward(self, x: torch.Tensor, exact: bool = False) -> torch.Tensor:
        if self.bias is not None:
            return ops.gemm_any_act(x, self.weight, bias=self.bias, exact=exact)
        return ops.gemm_any(x, self.weight, exact=exact)


class OutputLayerNorm(nn.Module):
    def __init__(self, width: int, eps: float):
        super().__init__()
        self.eps = eps
        self.weight, self.bias = _vector(width, 1.0), _vector(width)

    def add_to(self, residual: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
        """residual += LN(y), in place."""
        return ops.layernorm_f32(y, self.weight, self.bias, self.eps, add_to=residual)

    def forward(self, y: torch.Tensor) -> torch.Tensor:
        return ops.layernorm_f32(y, self.weight, self.bias, self.eps)


class SlidingWindowAttention(nn.Module):
    """mixes_values: "first" (this layer's values are what later layers mix in), "later" (mixes them in with its
    own coefficient) or None."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int, scale: float, eps: float,
                 mixes_values: str | None = None):
        super().__init__()
        assert heads % kv_heads == 0
        self.H, self.G, self.D, self.Dv, self.window, self.scale, self.eps = heads, kv_heads, dim, vdim, window, scale, eps
        self.mixes_values = mixes_values
        self.qkvg = MergedRows(width, {"q": heads * dim, "k": kv_heads * dim, "v": kv_heads * vdim, "g": heads * vdim})
        self.q_norm, self.k_norm = _vector(heads * dim, 1.0), _vector(kv_heads * dim, 1.0)
        self.vmix = _vector(1)
        self.o = _matrix(width, heads * vdim)
        self.k_cache = self.v_cache = torch.tensor([])

    def cache_shapes(self, num_blocks: int, block_size: int):
        return (num_blocks, self.G, block_size, self.D), (num_blocks, self.G, block_size, self.Dv)

    def forward(self, x: torch.Tensor, v_first: torch.Tensor | None):
        ctx, m = get_context(), self.qkvg
        y = m(x)
        (qo, _), (ko, _), (vo, nv), (go, _) = m.offsets["q"], m.offsets["k"], m.offsets["v"], m.offsets["g"]
        mix_in = v_first if self.mixes_values == "later" else None
        ops.swa_prepare(y, qo, ko, vo, self.q_norm, self.k_norm, self.eps, mix_in, self.vmix if mix_in is not None else None,
                        self.k_cache, self.v_cache, ctx.slot_mapping, self.H, self.G, self.D, self.Dv, ctx.block_size)
        o = ops.swa_attention(m.cols(y, "q"), self.k_cache, self.v_cache, ctx.block_tables, ctx.cu_seqlens_q, ctx.kv_lens,
                              self.H, self.G, self.D, self.Dv, ctx.block_size, self.window, self.scale,
                              gate=m.cols(y, "g"))
        return ops.gemm_any(o, self.o), (y[:, vo:vo + nv] if self.mixes_values == "first" else v_first)


class ChannelDeltaMixer(nn.Module):
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, decay_rank: int,
                 gate_rank: int, eps: float):
        super().__init__()
        assert heads % kv_heads == 0
        self.H, self.G, self.D, self.Dv, self.taps, self.eps = heads, kv_heads, dim, vdim, taps, eps
        parts = {"q": kv_heads * dim, "k": kv_heads * dim, "v": heads * vdim}
        self.qkv = MergedRows(width, parts)
        self.conv = MergedRows(taps, parts, dtype=torch.float32)  # [channels, taps]: per-channel filters, same row ranges
        self.low = MergedRows(width, {"a1": decay_rank, "g1": gate_rank, "b": heads})
        self.a2, self.g2 = _matrix(heads * dim, decay_rank), _matrix(heads * vdim, gate_rank)
        self.dt_bias, self.A_log, self.norm = _vector(heads * dim), _vector(heads), _vector(vdim, 1.0)
        self.o = _matrix(width, heads * vdim)
        self.state = self.conv_state = torch.tensor([])

    def state_shapes(self, n_slots: int):
        return ((n_slots, ops.channel_delta_state_elems(self.H, self.D, self.Dv)),
                (n_slots, max(self.taps - 1, 1), self.qkv.weight.shape[0]))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        cu, kv, slots = ctx.cu_seqlens_q, ctx.kv_lens, ctx.state_slots
        pre = self.qkv(x)
        qkv = ops.causal_conv_advance(pre, self.conv.weight, self.conv_state, cu, kv, slots, ctx.max_seqlen_q, silu=True)
        low = self.low(x)
        decay_pre = ops.gemm_any(self.low.cols(low, "a1"), self.a2)
        gate_pre = ops.gemm_any(self.low.cols(low, "g1"), self.g2)
        off = self.qkv.offsets
        o = ops.channel_delta(qkv, off["q"][0], off["k"][0], off["v"][0], self.low.cols(low, "b"), decay_pre, self.dt_bias,
                              self.A_log, gate_pre, self.norm, self.state, cu, kv, slots, self.H, self.G, self.D, self.Dv,
                              self.eps)
        return ops.gemm_any(o, self.o)


class GroupedSparseMLP(nn.Module):
    """score: "softmax" over the router's outputs or each output's own "sigmoid"; group_value: a group of neighbouring
    outputs is ranked by its best choice score ("max") or by the sum of its two best ("top2")."""

    def __init__(self, width: int, ff: int, experts: int, identity: int, top_k: int, groups: int, keep: int,
                 score: str = "softmax", group_value: str = "max"):
        super().__init__()
        self.E, self.n_out, self.top_k, self.groups, self.keep = experts, experts + identity, top_k, groups, keep
        self.score_kind = {"softmax": _C.ROUTE_SOFTMAX, "sigmoid": _C.ROUTE_SIGMOID}[score]
        self.group_kind = {"max": _C.ROUTE_GROUP_MAX, "top2": _C.ROUTE_GROUP_TOP2}[group_value]
        assert self.n_out % groups == 0 and 1 <= keep <= groups and top_k <= keep * (self.n_out // groups)
        self.router = _matrix(self.n_out, width)
        self.correction = _vector(self.n_out)
        self.gate, self.up, self.down = _matrix(experts, ff, width), _matrix(experts, ff, width), _matrix(experts, width, ff)
        for p in (self.gate, self.up, self.down):
            p.weight_loader = lambda param, tensor, expert: param.data[expert].copy_(tensor)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        z = ops.gemm_any(x, self.router, exact=True)  # router logits in true 32-bit in every serving mode
        ids, wts = ops.route_grouped(z, self.correction, self.top_k, self.groups, self.keep, self.score_kind,
                                     self.group_kind)
        offsets, pair_token, pair_index = ops.moe_sort(ids, self.n_out)
        P = ids.numel()
        act = ops.gemm_any_grouped(x, pair_token, self.gate, self.up, offsets, P, None, P)
        y = ops.gemm_any_grouped(act, None, self.down, None, offsets, P, pair_index, P)
        return ops.moe_combine_f32(y, x, ids, wts, self.E)


# ---------------------------------------------------------------------------------------------------------------------
# pre-norm families with a depth-mixed residual stream
# ---------------------------------------------------------------------------------------------------------------------
_ACTS = {"silu": _C.ACT_SILU, "gelu_tanh": _C.ACT_GELU_TANH, "gelu": _C.ACT_GELU_ERF, "sigmoid": _C.ACT_SIGMOID, None: _C.ACT_NONE}
CAUSAL = 2 ** 31 - 1   # "window" of plain causal attention


def rotary_inv_freq(dims: int, base: float) -> torch.Tensor:
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)] or [0.0]
    return torch.tensor(f, dtype=torch.float64).to(torch.float32)


class DepthMixedResidual:
    """The residual stream of one step: slot 0 holds the embedding rows, slot i + 1 layer i's result
    X_{i+1} = a + m f1(n1(a)) + m f2(n2(.)), where a - what layer i reads - is the weighted sum of the slots 0..i with the
    previous layer's coefficients (layer 0 reads slot 0 itself).  The sum for layer i + 1 is written straight into slot
    i + 2 and becomes X_{i+2} by the in-place residual updates.  One launch per layer boundary folds the last residual
    update, the weighted sum and the next layer's first norm."""

    def __init__(self, rows: int, width: int, n_layers: int, mult: float, eps: float, unit: torch.Tensor, shift: float = 1.0):
        """unit: a device tensor holding 1.0 (the first layer's only coefficient)"""
        self.stack = torch.empty((n_layers + 2, rows, width), dtype=torch.float32, device=unit.device)  # slot 0: the caller's
        self.n, self.mult, self.eps, self.shift = 1, mult, eps, shift
        self._one = unit

    @property
    def current(self) -> torch.Tensor:
        return self.stack[self.n]

    def begin(self, norm_w: torch.Tensor) -> torch.Tensor:
        """-> n(slot 0) for the first layer"""
        return ops.depth_mix_f32(self.stack, 1, self._one, None, 0.0, norm_w, self.eps, self.shift)

    def add_and_norm(self, y: torch.Tensor, norm_w: torch.Tensor | None):
        """current += m * y; -> its norm (None without a weight)"""
        return ops.add_rmsnorm_f32(self.current, y, self.mult, norm_w, self.eps, self.shift)

    def next_layer(self, y: torch.Tensor | None, coef: torch.Tensor, norm_w: torch.Tensor | None):
        """current += m * y (the layer's last sublayer); the weighted sum of all results so far opens the next slot;
        -> its norm with the next layer's first norm weight (None after the last layer)"""
        self.n += 1
        return ops.depth_mix_f32(self.stack, self.n, coef, y, self.mult, norm_w, self.eps, self.shift)


class MinGRUMixer(nn.Module):
    """z = sigmoid(W_z h + b_z), u = W_x h + b_x, c = u + 1/2 (u >= 0) | sigmoid(u); S <- (1 - z) S + z c per channel;
    out = W_o (S * silu(W_g h)).  The state [slots, width] is fp32."""

    def __init__(self, width_in: int, width: int):
        super().__init__()
        self.n = width
        self.zxg = MergedRows(width_in, {"z": width, "x": width, "g": width}, bias=True)
        self.o = _matrix(width_in, width)
        self.state = torch.tensor([])

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx, off = get_context(), self.zxg.offsets
        y = self.zxg(h)
        s = ops.mingru_scan(y, off["z"][0], off["x"][0], off["g"][0], self.n, self.state, ctx.cu_seqlens_q, ctx.kv_lens,
                            ctx.state_slots, ctx.max_seqlen_q)
        return ops.gemm_any(s, self.o)


class LatentAttention(nn.Module):
    """[c | r] = W_dkv h; c <- rms(c) * w_c; k_h = [W_uk,h c | rot(r)], v_h = W_uv,h c; q_h = [q_h' | rot(q_h'')].
    Cached per token: [c | rot(r)] only - ONE key/value row for all heads.  Scores and outputs are formed in the latent
    space: q_h'.(W_uk,h c) = (W_uk,h^T q_h').c, sum_j p_j W_uv,h c_j = W_uv,h (sum_j p_j c_j), so the attention is
    multi-query attention with key rows [c | r] of C + R channels whose first C channels are also the values; the two
    per-head projections around it are batched GEMMs over head-major rows."""

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, rot_dims: int,
                 rot_base: float, scale: float, eps: float, q_rank: int = 0, gate: bool = True, sink: bool = False):
        """q_rank > 0: the queries come through a latent of their own, q = W_uq rms(W_dq h) * w_q (the down-projection
        rides with the key/value one); gate: sigmoid output gate W_g h; sink: a learned logit per head in the softmax's
        denominator.  rot_dim = 0: no rotated part - nothing in the layer depends on positions."""
        super().__init__()
        assert 0 <= rot_dims <= rot_dim and rot_dims % 2 == 0
        self.H, self.D, self.R, self.Dv, self.C, self.Q = heads, dim, rot_dim, vdim, kv_rank, q_rank
        self.rot_dims, self.rot_base, self.scale, self.eps = rot_dims, rot_base, scale, eps
        # base^(-2 i / dims) in double, rounded once (a buffer, not a checkpoint tensor)
        self.register_buffer("inv_freq", rotary_inv_freq(rot_dims, rot_base), persistent=False)
        parts = {"dq": q_rank} if q_rank else {"q": heads * (dim + rot_dim)}
        parts["dkv"] = kv_rank + rot_dim
        if gate:
            parts["g"] = heads * vdim
        self.gated = gate
        self.qcg = MergedRows(width, parts)
        if q_rank:
            self.q_norm = _vector(q_rank, 1.0)
            self.uq = _matrix(heads * (dim + rot_dim), q_rank)
        self.sink = _vector(heads) if sink else None
        self.c_norm = _vector(kv_rank, 1.0)
        self.uk_t = _matrix(heads, kv_rank, dim)   # W_uk,h transposed: the query-side projection into the latent space
        self.uv = _matrix(heads, vdim, kv_rank)
        self.uk_t.weight_loader = lambda p, t: p.data.copy_(t.view(heads, dim, kv_rank).transpose(1, 2))
        self.uv.weight_loader = lambda p, t: p.data.copy_(t.view(heads, vdim, kv_rank))
        self.o = _matrix(width, heads * vdim)
        self.cache = torch.tensor([])

    def cache_shape(self, num_blocks: int, block_size: int):
        return (num_blocks, 1, block_size, self.C + self.R)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx, m = get_context(), self.qcg
        H, D, R, Dv, C = self.H, self.D, self.R, self.Dv, self.C
        y = m(h)
        if self.Q:   # queries through their own latent: norm of the down-projection's columns, then the up-projection
            q, q_off = ops.gemm_any(ops.add_rmsnorm_f32(m.cols(y, "dq"), None, 0.0, self.q_norm, self.eps), self.uq), 0
        else:
            q, q_off = y, m.offsets["q"][0]
        qx = torch.empty((h.shape[0], H * (C + R)), dtype=torch.float32, device=h.device)
        ops.latent_prepare(y, q, q_off, m.offsets["dkv"][0], H, D, R, C, self.rot_dims, self.inv_freq, self.c_norm,
                           self.eps, ctx.cu_seqlens_q, ctx.kv_lens, self.cache, ctx.slot_mapping, qx)
        ops.gemm_any_batched(q[:, q_off:q_off + H * (D + R)], D + R, self.uk_t, qx, C + R)
        o = ops.paged_attention_f32(qx, self.cache, self.cache, C + R, ctx.block_tables, ctx.cu_seqlens_q, ctx.kv_lens, H, 1,
                                    C + R, C, ctx.block_size, CAUSAL, self.scale, _C.BIAS_NONE, sink=self.sink)
        ov = torch.empty((h.shape[0], H * Dv), dtype=torch.float32, device=h.device)
        ops.gemm_any_batched(o, C, self.uv, ov, Dv, gate=m.cols(y, "g") if self.gated else None, gate_batch=Dv)
        return ops.gemm_any(ov, self.o)


class BiasedAttention(nn.Module):
    """s_ij = scale * t(i) q_i . k_j - r1_h ln(1 + r2_h (i - j)), t(p) = 1 + coef ln(floor((p + 1) / every) + 1)
    (every < 1: no temperature); causal, grouped key/value heads of separate key and value sizes, no rotation."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, temp_coef: float = 0.0,
                 temp_every: int = 0):
        super().__init__()
        assert heads % kv_heads == 0
        self.H, self.G, self.D, self.Dv, self.scale = heads, kv_heads, dim, vdim, scale
        self.temp_coef, self.temp_every = temp_coef, temp_every
        self.qkv = MergedRows(width, {"q": heads * dim, "k": kv_heads * dim, "v": kv_heads * vdim})
        self.r1, self.r2 = _vector(heads), _vector(heads)
        self.o = _matrix(width, heads * vdim)
        self.k_cache = self.v_cache = torch.tensor([])

    def cache_shapes(self, num_blocks: int, block_size: int):
        return (num_blocks, self.G, block_size, self.D), (num_blocks, self.G, block_size, self.Dv)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx, m = get_context(), self.qkv
        y = m(h)
        ops.kv_store_temp(y, m.offsets["q"][0], m.offsets["k"][0], m.offsets["v"][0], self.temp_coef, self.temp_every,
                          ctx.cu_seqlens_q, ctx.kv_lens, self.k_cache, self.v_cache, ctx.slot_mapping, self.H, self.G,
                          self.D, self.Dv, ctx.block_size)
        o = ops.paged_attention_f32(m.cols(y, "q"), self.k_cache, self.v_cache, self.Dv, ctx.block_tables, ctx.cu_seqlens_q,
                                    ctx.kv_lens, self.H, self.G, self.D, self.Dv, ctx.block_size, CAUSAL, self.scale,
                                    _C.BIAS_LOG, self.r1, self.r2)
        return ops.gemm_any(o, self.o)


class GatedDenseMLP(nn.Module):
    def __init__(self, width: int, ff: int, act: str = "gelu_tanh"):
        super().__init__()
        self.act = _ACTS[act]
        self.gate, self.up, self.down = _matrix(ff, width), _matrix(ff, width), _matrix(width, ff)
        self.gate_b, self.up_b, self.down_b = _vector(ff), _vector(ff), _vector(width)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        a = ops.gemm_any_act(h, self.gate, bias=self.gate_b, act=self.act, w2=self.up, bias2=self.up_b)
        return ops.gemm_any_act(a, self.down, bias=self.down_b)


class SharedSparseMLP(nn.Module):
    """Router logits in true 32-bit; the `top_k` largest, weights = softmax over them; experts W_d act(W_u h) without
    biases; shared_ff > 0: a shared expert of the same form for every token, times sigmoid(w_sg . h) - that gate's row
    rides behind the router's rows in one projection."""

    def __init__(self, width: int, ff: int, experts: int, top_k: int, shared_ff: int = 0, act: str = "gelu"):
        super().__init__()
        assert 1 <= top_k <= experts
        self.E, self.top_k, self.act, self.shared = experts, top_k, _ACTS[act], shared_ff > 0
        self.router = MergedRows(width, {"router": experts, "sg": 1} if self.shared else {"router": experts})
        self.up, self.down = _matrix(experts, ff, width), _matrix(experts, width, ff)
        for p in (self.up, self.down):
            p.weight_loader = lambda param, tensor, expert: param.data[expert].copy_(tensor)
        if self.shared:
            self.shared_up, self.shared_down = _matrix(shared_ff, width), _matrix(width, shared_ff)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        z = self.router(h, exact=True)
        ids, wts = ops.route_topk(z, self.E, self.top_k)
        offsets, pair_token, pair_index = ops.moe_sort(ids, self.E)
        P = ids.numel()
        a = ops.gemm_any_grouped_act(h, pair_token, self.up, None, self.act, offsets, P, None, P)
        y = ops.gemm_any_grouped_act(a, None, self.down, None, _C.ACT_NONE, offsets, P, pair_index, P)
        if not self.shared:
            return ops.moe_combine_shared(y, ids, wts, h.shape[1])
        sh = ops.gemm_any(ops.gemm_any_act(h, self.shared_up, act=self.act), self.shared_down)
        return ops.moe_combine_shared(y, ids, wts, h.shape[1], sh, z[:, self.E:])


# ---------------------------------------------------------------------------------------------------------------------
# sandwich-normed families: gated residual branches, an input convolution, linear attention with a decayed state
# ---------------------------------------------------------------------------------------------------------------------
class InputConvolution(nn.Module):
    """u = h + conv(h), conv(h)_t[c] = sum_j w[c, j] h_{t - (taps - 1) + j}[c] with zeros before the sequence's start.
    The last taps - 1 rows of h live in the sequence's state slot `state` [slots, taps - 1, width]."""

    def __init__(self, width: int, taps: int):
        super().__init__()
        assert 1 <= taps <= 17
        self.taps = taps
        self.weight = nn.Parameter(torch.zeros(width, taps, dtype=torch.float32), requires_grad=False)
        self.state = torch.tensor([])

    def state_shape(self, n_slots: int):
        return (n_slots, max(self.taps - 1, 1), self.weight.shape[0])

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        cu, kv, slots = ctx.cu_seqlens_q, ctx.kv_lens, ctx.state_slots
        return ops.causal_conv_advance(h, self.weight, self.state, cu, kv, slots, ctx.max_seqlen_q, silu=False, add_input=True)


class GatedOutputNorm(nn.Module):
    """x <- x + rms(sigmoid(W_g h + b_g) * f(h)) * w, h being what the sublayer f was handed."""

    def __init__(self, width: int, eps: float):
        super().__init__()
        self.eps = eps
        self.gate, self.gate_b, self.weight = _matrix(width, width), _vector(width), _vector(width, 1.0)

    def gate_of(self, h: torch.Tensor) -> torch.Tensor:
        """-> W_g h + b_g (the sigmoid is taken where the gate is applied)"""
        return ops.gemm_any_act(h, self.gate, bias=self.gate_b)

    def add_to(self, residual: torch.Tensor, y: torch.Tensor, gate_pre: torch.Tensor, next_norm: torch.Tensor | None):
        """residual += rms(y * sigmoid(gate_pre)) * w in place; -> rms(residual) * next_norm (None without one)"""
        return ops.gated_norm_add_f32(residual, y, gate_pre, self.weight, self.eps, next_norm)


class _LinearAttentionState(nn.Module):
    def state_shape(self, n_slots: int):
        return (n_slots, ops.linear_attention_state_elems(self.H, self.D, self.Dv))


class HeadDecayLinearAttention(_LinearAttentionState):
    """q = silu(W_q u), k = silu(W_k u), v = silu(W_v u); per head S <- decay_h S + k v^T, o = S^T q; the heads' read-outs
    are RMS-normed TOGETHER (weight [heads * vdim]), times sigmoid(W_g u), then W_o.  fp32 state per sequence slot."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay, eps: float):
        super().__init__()
        assert len(decay) == heads
        self.H, self.D, self.Dv, self.eps = heads, dim, vdim, eps
        self.qkvg = MergedRows(width, {"q": heads * dim, "k": heads * dim, "v": heads * vdim, "g": heads * vdim})
        self.register_buffer("decay", torch.tensor([float(d) for d in decay], dtype=torch.float64).to(torch.float32),
                             persistent=False)
        self.norm = _vector(heads * vdim, 1.0)
        self.o = _matrix(width, heads * vdim)
        self.state = torch.tensor([])

    def forward(self, u: torch.Tensor) -> torch.Tensor:
        ctx, m = get_context(), self.qkvg
        y = m(u)
        off = m.offsets
        o = ops.linear_attention(y, off["q"][0], off["k"][0], off["v"][0], (_C.ACT_SILU,) * 3, _C.DECAY_HEAD, self.decay, None,
                                 None, m.cols(y, "g"), self.norm, 1, self.state, ctx.cu_seqlens_q, ctx.kv_lens,
                                 ctx.state_slots, self.H, self.D, self.Dv, self.eps)
        return ops.gemm_any(o, self.o)


class ForgetGateLinearAttention(_LinearAttentionState):
    """q = silu(W_q u), v = W_v u, f = l + (1 - l) sigmoid(W_f u + b_f) with a lower bound l per channel; per head
    S <- diag(f) S + (1 - f) v^T, o = S^T q; each head's read-out is RMS-normed over its value channels (one weight [vdim]
    for all heads), then W_o.  fp32 state per sequence slot."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, eps: float):
        super().__init__()
        self.H, self.D, self.Dv, self.eps = heads, dim, vdim, eps
        self.qfv = MergedRows(width, {"q": heads * dim, "f": heads * dim, "v": heads * vdim})
        self.f_bias, self.lower, self.norm = _vector(heads * dim), _vector(heads * dim), _vector(vdim, 1.0)
        self.o = _matrix(width, heads * vdim)
        self.state = torch.tensor([])

    def forward(self, u: torch.Tensor) -> torch.Tensor:
        ctx, m = get_context(), self.qfv
        y = m(u)
        off = m.offsets
        o = ops.linear_attention(y, off["q"][0], off["f"][0], off["v"][0], (_C.ACT_SILU, _C.ACT_NONE, _C.ACT_NONE),
                                 _C.DECAY_FORGET, None, self.f_bias, self.lower, None, self.norm, self.H, self.state,
                                 ctx.cu_seqlens_q, ctx.kv_lens, ctx.state_slots, self.H, self.D, self.Dv, self.eps)
        return ops.gemm_any(o, self.o)


# ---------------------------------------------------------------------------------------------------------------------
# looped pre-norm families: rotated window attention with its options, retention, experts weighted on their input
# ---------------------------------------------------------------------------------------------------------------------
def rotary_table(dims: int, base: float, scaling: dict | None = None):
    """-> (frequencies [dims / 2] fp32, amplitude of cos and sin).  f_i = base^(-2 i / dims), computed in double and
    rounded once.  scaling {factor, original, fast, slow}: with c(r) = dims ln(original / (2 pi r)) / (2 ln base) - the pair
    that turns r times over `original` positions - the pairs up to floor c(fast) keep their frequency, those from
    ceil c(slow) on are divided by `factor`, a linear ramp in between; cos and sin are multiplied by 0.1 ln(factor) + 1."""
    import math

    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    amp = 1.0
    if scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def c(r):
            return dims * math.log(original / (2 * math.pi * r)) / (2 * math.log(float(base)))

        lo = max(math.floor(c(float(scaling["fast"]))), 0)
        hi = min(math.ceil(c(float(scaling["slow"]))), dims - 1)
        ramp = [min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)]
        f = [fi / factor * r + fi * (1 - r) for fi, r in zip(f, ramp)]
        amp = 0.1 * math.log(factor) + 1.0
    return torch.tensor(f or [0.0], dtype=torch.float64).to(torch.float32), amp


class RotaryWindowAttention(nn.Module):
    """The attention itself, on projections its owner made (`parts`: name -> rows of the q / k / v projections, to be laid
    out next to each other in this order).  conv_taps > 0: q, k and v first pass a causal convolution per channel (filters
    `conv.weight` [channels, taps], no activation), whose last taps - 1 inputs are the sequence's state.  Then q and k are
    rotated (pairs 2i, 2i + 1 of the first rot_dims channels), unit_norm: each head divided by its root mean square;
    s = scale q.k, softcap > 0: s <- softcap tanh(s / softcap); keys 0 <= i - j < window; softmax, sink: with
    exp(sink_h) in the denominator; talk: the heads' weights are mixed, p'_h = sum_g talk[h, g] p_g, before head h applies
    them to the values of its own key/value head.

    The mixing is linear in the weights, so it is done on read-outs: every query head's weights are applied to the values
    of ALL key/value heads (the value pages hold a token's heads side by side as ONE wide head, read in chunks of at most
    256 channels), then out_h = sum_g talk[h, g] o[g, kv(h)]."""

    def __init__(self, heads: int, kv_heads: int, dim: int, vdim: int, window: int, scale: float, eps: float,
                 rot_dims: int, rot_base: float, rot_scaling: dict | None = None, unit_norm: bool = False,
                 sink: bool = False, softcap: float = 0.0, conv_taps: int = 0, talk: bool = False):
        super().__init__()
        assert heads % kv_heads == 0 and 0 <= rot_dims <= dim and rot_dims % 2 == 0
        self.H, self.G, self.D, self.Dv = heads, kv_heads, dim, vdim
        self.window, self.scale, self.eps, self.unit_norm, self.softcap = window, scale, eps, unit_norm, softcap
        self.rot_dims = rot_dims
        freq, self.rot_amp = rotary_table(rot_dims, rot_base, rot_scaling) if rot_dims else (torch.zeros(1, dtype=torch.float32), 1.0)
        self.register_buffer("inv_freq", freq, persistent=False)
        self.parts = {"q": heads * dim, "k": kv_heads * dim, "v": kv_heads * vdim}
        self.sink = _vector(heads) if sink else None
        self.talk = nn.Parameter(torch.eye(heads, dtype=torch.float32), requires_grad=False) if talk else None
        self.conv = MergedRows(conv_taps, self.parts, dtype=torch.float32) if conv_taps else None
        self.k_cache, self.v_cache, self.conv_state = [], [], []   # one per lane
        # value heads read together by one launch when the weights are mixed
        self.chunk = max(1, min(kv_heads, 256 // vdim)) if talk else 0

    @property
    def out_features(self) -> int:
        return self.H * self.Dv

    def cache_shapes(self, num_blocks: int, block_size: int):
        v = (num_blocks, 1, block_size, self.G * self.Dv) if self.talk is not None else (num_blocks, self.G, block_size, self.Dv)
        return (num_blocks, self.G, block_size, self.D), v

    def conv_state_shape(self, n_slots: int):
        return (n_slots, max(self.conv.weight.shape[1] - 1, 1), self.conv.weight.shape[0]) if self.conv is not None else None

    def attend(self, y: torch.Tensor, q_off: int, lane: int, out: torch.Tensor, out_scale: float = 1.0) -> None:
        """y: rows holding q | k | v from column q_off on; out [rows, >= heads * vdim] receives out_scale * read-out."""
        ctx = get_context()
        H, G, D, Dv = self.H, self.G, self.D, self.Dv
        n = H * D + G * D + G * Dv
        if self.conv is not None:
            y = ops.causal_conv_advance(y[:, q_off:q_off + n], self.conv.weight, self.conv_state[lane], ctx.cu_seqlens_q,
                                        ctx.kv_lens, ctx.state_slots, ctx.max_seqlen_q)
            q_off = 0
        k_off, v_off = q_off + H * D, q_off + H * D + G * D
        kc, vc = self.k_cache[lane], self.v_cache[lane]
        ops.rotary_store(y, q_off, k_off, v_off, H, G, D, self.rot_dims, _C.ROT_INTERLEAVED, self.inv_freq, self.rot_amp,
                         self.unit_norm, self.eps, 1.0, ctx.cu_seqlens_q, ctx.kv_lens, kc, vc, ctx.slot_mapping, ctx.block_size)
        q = y[:, q_off:q_off + H * D]
        if self.talk is None:
            ops.paged_attention_f32(q, kc, vc, Dv, ctx.block_tables, ctx.cu_seqlens_q, ctx.kv_lens, H, G, D, Dv,
                                    ctx.block_size, self.window, self.scale, _C.BIAS_NONE, sink=self.sink,
                                    softcap=self.softcap, out=out)
            if out_scale != 1.0:
                out.mul_(out_scale)
            return
        for c0 in range(0, G, self.chunk):
            nc = min(self.chunk, G - c0)
            o = ops.paged_attention_f32(q, kc, vc, G * Dv, ctx.block_tables, ctx.cu_seqlens_q, ctx.kv_lens, H, G, D, nc * Dv,
                                        ctx.block_size, self.window, self.scale, _C.BIAS_NONE, sink=self.sink,
                                        softcap=self.softcap, value_heads=1, v_offset=c0 * Dv)
            ops.head_mix(o, self.talk, H, G, Dv, c0, nc, out, out_scale)


class Retention(nn.Module):
    """q, k rotated (pairs i, i + rot_dims / 2 of the first rot_dims channels), k <- k dim^(-1/2); per head
    S <- decay_h S + k v^T, o = S^T q (fp32 state per sequence slot and lane, no softmax, no denominator); each head's o
    divided by its root mean square, times silu(g)."""

    def __init__(self, heads: int, dim: int, vdim: int, decay, eps: float, rot_dims: int, rot_base: float,
                 rot_scaling: dict | None = None):
        super().__init__()
        assert len(decay) == heads and 0 <= rot_dims <= dim and rot_dims % 2 == 0
        self.H, self.D, self.Dv, self.eps, self.rot_dims = heads, dim, vdim, eps, rot_dims
        freq, self.rot_amp = rotary_table(rot_dims, rot_base, rot_scaling) if rot_dims else (torch.zeros(1, dtype=torch.float32), 1.0)
        self.register_buffer("inv_freq", freq, persistent=False)
        self.register_buffer("decay", torch.tensor([float(d) for d in decay], dtype=torch.float64).to(torch.float32),
                             persistent=False)
        self.parts = {"q": heads * dim, "k": heads * dim, "v": heads * vdim, "g": heads * vdim}
        self.state = []   # one per lane

    @property
    def out_features(self) -> int:
        return self.H * self.Dv

    def state_shape(self, n_slots: int):
        return (n_slots, ops.linear_attention_state_elems(self.H, self.D, self.Dv))

    def scan(self, y: torch.Tensor, q_off: int, lane: int, out: torch.Tensor, out_scale: float = 1.0) -> None:
        """y: rows holding q | k | v | g from column q_off on (q and k are rotated in place); out [rows, heads * vdim]."""
        ctx = get_context()
        H, D, Dv = self.H, self.D, self.Dv
        k_off, v_off, g_off = q_off + H * D, q_off + 2 * H * D, q_off + 2 * H * D + H * Dv
        ops.rotary_store(y, q_off, k_off, v_off, H, H, D, self.rot_dims, _C.ROT_HALVES, self.inv_freq, self.rot_amp, False,
                         self.eps, D ** -0.5, ctx.cu_seqlens_q, ctx.kv_lens)
        ops.linear_attention(y, q_off, k_off, v_off, (_C.ACT_NONE,) * 3, _C.DECAY_HEAD, self.decay, None, None, None, None, H,
                             self.state[lane], ctx.cu_seqlens_q, ctx.kv_lens, ctx.state_slots, H, D, Dv, self.eps, out=out)
        ops.head_norm_gate(out, y[:, g_off:g_off + H * Dv], _C.ACT_SILU, None, H, Dv, self.eps, out_scale)


class SinkAttentionMixer(nn.Module):
    """W_o attention(W_q h, W_k h, W_v h) with a RotaryWindowAttention as the attention."""

    def __init__(self, width: int, attention: RotaryWindowAttention):
        super().__init__()
        self.attn = attention
        self.qkv = MergedRows(width, attention.parts)
        self.o = _matrix(width, attention.out_features)

    def forward(self, h: torch.Tensor, lane: int = 0) -> torch.Tensor:
        y = self.qkv(h)
        out = torch.empty((h.shape[0], self.attn.out_features), dtype=torch.float32, device=h.device)
        self.attn.attend(y, 0, lane, out)
        return ops.gemm_any(out, self.o)


class ParallelMixers(nn.Module):
    """left_scale * W_ol attention(h) + right_scale * W_or retention(h): the seven projections of h are ONE product, the
    two read-outs are written, already scaled, side by side into one buffer, and [W_ol | W_or] is ONE output projection."""

    def __init__(self, width: int, left: RotaryWindowAttention, right: Retention, left_scale: float, right_scale: float):
        super().__init__()
        self.left, self.right, self.left_scale, self.right_scale = left, right, left_scale, right_scale
        parts = {f"left.{n}": r for n, r in left.parts.items()}
        parts.update({f"right.{n}": r for n, r in right.parts.items()})
        self.proj = MergedRows(width, parts)
        nl, nr = left.out_features, right.out_features
        self.o = _matrix(width, nl + nr)
        spans = {"left": (0, nl), "right": (nl, nr)}

        def load_o(param, tensor, side):
            off, n = spans[side]
            assert tensor.shape[1] == n, (side, tuple(tensor.shape), n)
            param.data[:, off:off + n].copy_(tensor)
        self.o.weight_loader = load_o

    def forward(self, h: torch.Tensor, lane: int = 0) -> torch.Tensor:
        y = self.proj(h)
        nl, nr = self.left.out_features, self.right.out_features
        out = torch.empty((h.shape[0], nl + nr), dtype=torch.float32, device=h.device)
        self.left.attend(y, self.proj.offsets["left.q"][0], lane, out[:, :nl], self.left_scale)
        self.right.scan(y, self.proj.offsets["right.q"][0], lane, out[:, nl:], self.right_scale)
        return ops.gemm_any(out, self.o)


class InputWeightedSparseMLP(nn.Module):
    """Router logits in true 32-bit, scores = sigmoid; the top_k largest; out = sum_k expert_k(s_k h) - the score
    multiplies the expert's input (experts have no biases: s (W h) = W (s h), so it is applied to the first projections'
    accumulators).  Expert: g = min(W_g x, limit), u = clamp(W_u x, -limit, limit), W_d (g sigmoid(1.702 g) (u + 1))."""

    def __init__(self, width: int, ff: int, experts: int, top_k: int, limit: float):
        super().__init__()
        assert 1 <= top_k <= experts and limit > 0
        self.E, self.top_k, self.limit = experts, top_k, limit
        self.router = _matrix(experts, width)
        self.register_buffer("no_correction", torch.zeros(experts, dtype=torch.float32), persistent=False)
        self.gate, self.up, self.down = _matrix(experts, ff, width), _matrix(experts, ff, width), _matrix(experts, width, ff)
        for p in (self.gate, self.up, self.down):
            p.weight_loader = lambda param, tensor, expert: param.data[expert].copy_(tensor)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        z = ops.gemm_any(h, self.router, exact=True)
        ids, wts = ops.route_grouped(z, self.no_correction, self.top_k, 1, 1, _C.ROUTE_SIGMOID, _C.ROUTE_GROUP_MAX)
        offsets, pair_token, pair_index = ops.moe_sort(ids, self.E)
        P = ids.numel()
        a = ops.gemm_any_grouped_glu(h, pair_token, self.gate, self.up, _C.ACT_CLAMPED_GLU, self.limit, wts, pair_index,
                                     offsets, P, None, P)
        y = ops.gemm_any_grouped(a, None, self.down, None, offsets, P, pair_index, P)
        return ops.moe_combine_shared(y, ids, None, h.shape[1])

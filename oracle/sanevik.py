"""Plain, slow statement of the Sanevik design (torch on CPU, float64 by default): one function per mechanism.

TEST INFRASTRUCTURE: nothing of the product path imports this file and it imports nothing of the product path.
One sequence at a time, whole, with dense [T, T] score matrices and Python loops over time for the recurrence.

Notation (W x means `x @ W.T`, weights stored [out, in]; t = position, counted from 0):

  norm          n(x; w) = x / sqrt(mean(x^2) + eps) * (1 + w);   u(x) = x / sqrt(mean(x^2) + eps)
  layer         x <- x + mixer(n(x; w_1));   x <- x + ff(n(x; w_2))            (a layer may have no feed-forward)
  order         layers [0, start), then `times` passes over [start, stop) with the same weights, then [stop, n);
                pass t begins with  x <- x + (t > 0 ? e : 0) + step[t],  e = the embedding rows
  rotation      angle a = t * f_i,  f_i = base^(-2 i / dims);  pairs (2i, 2i + 1) ["interleaved"] or (i, i + dims/2)
                ["halves"] of the first `dims` channels of a head:  (a, b) -> (a cos - b sin, b cos + a sin)
  long-context  with {factor, original, fast, slow}:  c(r) = dims ln(original / (2 pi r)) / (2 ln base),
  frequencies   lo = max(floor c(fast), 0),  hi = min(ceil c(slow), dims - 1),  ramp_i = clamp((i - lo) / max(hi - lo, .001), 0, 1),
                f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i);  cos and sin times 0.1 ln(factor) + 1
  attention     q, k rotated (interleaved), then u(q_h), u(k_h);  s_ij = scale q_i . k_j  for 0 <= i - j < window;
                p_ij = exp(s_ij) / (exp(sink_h) + sum_j' exp(s_ij'));  out = W_o concat_h(sum_j p_ij v_j)
  parallel      left_scale * left(h) + right_scale * right(h)
    left        q, k, v = conv(W h) per channel:  conv(u)_t = sum_{j < taps} w[:, j] u_{t - (taps - 1) + j},  zeros before t = 0
                q, k rotated (interleaved);  s = scale q.k;  s <- cap tanh(s / cap);  window;  p = softmax(s)
                p'_h = sum_g T[h, g] p_g;   out = W_o concat_h(sum_j p'_h,ij v_j)       (v of head h's own key/value head)
    right       q, k rotated (halves);  k <- k dim^(-1/2);  S_t = decay_h S_{t-1} + k_t v_t^T;  o_t = S_t^T q_t
                out = W_o (concat_h(u(o_h)) * silu(W_g h))
  sparse ff     s = sigmoid(W_r h);  the `top` largest;  out = sum_k expert_k(s_k h)
                expert(x) = W_d (g sigmoid(1.702 g) (u + 1)),  g = min(W_g x, limit),  u = clamp(W_u x, -limit, limit)
  output        logits = E n(x; w_final)      (E: the embedding table)
"""
from __future__ import annotations

import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * (1 + w)


def silu(z):
    return z * torch.sigmoid(z)


def rotary_frequencies(rot):
    """-> (f [dims / 2] as python floats, amplitude of cos and sin)"""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def c(r):
        return dims * math.log(original / (2 * math.pi * r)) / (2 * math.log(base))

    lo = max(math.floor(c(float(sc["fast"]))), 0)
    hi = min(math.ceil(c(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x, rot, layout):
    """x [T, heads, dim]; rotates the first rot.dims channels of every head; layout "interleaved" | "halves" """
    dims = int(rot["dims"])
    if dims == 0:
        return x
    T = x.shape[0]
    f, amp = rotary_frequencies(rot)
    ang = torch.arange(T, dtype=x.dtype).view(T, 1) * torch.tensor(f, dtype=x.dtype).view(1, -1)
    cos, sin = (torch.cos(ang) * amp).unsqueeze(1), (torch.sin(ang) * amp).unsqueeze(1)
    out = x.clone()
    if layout == "interleaved":
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * cos - b * sin
        out[..., 1:dims:2] = b * cos + a * sin
    else:
        a, b = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = a * cos - b * sin
        out[..., dims // 2:dims] = b * cos + a * sin
    return out


def visible(T, window):
    """[T, T] bool: key j is seen from position i"""
    d = torch.arange(T).view(T, 1) - torch.arange(T).view(1, T)
    ok = d >= 0
    if window is not None:
        ok &= d < window
    return ok


def window_of(m):
    return int(m["mask"]["size"]) if m.get("mask") else None


def short_conv(u, w):
    """u [T, C], w [C, taps] -> [T, C]"""
    T, taps = u.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u])
    out = torch.zeros_like(u)
    for j in range(taps):
        out = out + w[:, j] * padded[j:j + T]
    return out


def sink_attention_mixer(h, p, m, eps):
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms_unit(rotate((h @ p["q"].T).view(T, H, D), m["rot"], "interleaved"), eps)
    k = rms_unit(rotate((h @ p["k"].T).view(T, G, D), m["rot"], "interleaved"), eps)
    v = (h @ p["v"].T).view(T, G, Dv)
    k, v = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    s = torch.einsum("ihd,jhd->hij", q, k) * float(m["scale"])
    s = s.masked_fill(~visible(T, window_of(m)), float("-inf"))
    sink = p["sink"].view(H, 1, 1).expand(H, T, 1)
    pr = torch.softmax(torch.cat([s, sink], -1), -1)[..., :T]     # the sink takes weight and gives nothing
    o = torch.einsum("hij,jhd->ihd", pr, v).reshape(T, H * Dv)
    return o @ p["o"].T


def talking_attention_mixer(h, p, m, eps):
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q, k, v = h @ p["q"].T, h @ p["k"].T, h @ p["v"].T
    if m.get("conv"):
        q, k, v = short_conv(q, p["q.conv"]), short_conv(k, p["k.conv"]), short_conv(v, p["v.conv"])
    q = rotate(q.view(T, H, D), m["rot"], "interleaved")
    k = rotate(k.view(T, G, D), m["rot"], "interleaved").repeat_interleave(H // G, 1)
    v = v.view(T, G, Dv).repeat_interleave(H // G, 1)
    s = torch.einsum("ihd,jhd->hij", q, k) * float(m["scale"])
    cap = float(m.get("softcap") or 0.0)
    if cap > 0:
        s = cap * torch.tanh(s / cap)
    pr = torch.softmax(s.masked_fill(~visible(T, window_of(m)), float("-inf")), -1)
    if "talk" in p:
        pr = torch.einsum("hg,gij->hij", p["talk"], pr)
    o = torch.einsum("hij,jhd->ihd", pr, v).reshape(T, H * Dv)
    return o @ p["o"].T


def retention_mixer(h, p, m, eps):
    T = h.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    decay = torch.tensor([float(d) for d in m["decay"]], dtype=h.dtype)
    q = rotate((h @ p["q"].T).view(T, H, D), m["rot"], "halves")
    k = rotate((h @ p["k"].T).view(T, H, D), m["rot"], "halves") * D ** -0.5
    v = (h @ p["v"].T).view(T, H, Dv)
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    out = []
    for t in range(T):
        S = decay.view(H, 1, 1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    o = rms_unit(torch.stack(out), eps).reshape(T, H * Dv) * silu(h @ p["g"].T)
    return o @ p["o"].T


def parallel_mixer(h, p, m, eps):
    left = talking_attention_mixer(h, sub(p, "left."), m["left"], eps)
    right = retention_mixer(h, sub(p, "right."), m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def route(h, p, r):
    """-> (chosen experts [T, top], their weights [T, top])"""
    s = torch.sigmoid(h @ p["router"].T)
    idx = torch.topk(s, int(r["top"]), dim=-1).indices
    return idx, torch.gather(s, 1, idx)


def expert_ff(x, p, e, limit):
    g = torch.clamp(x @ p[f"e{e}.gate"].T, max=limit)
    u = torch.clamp(x @ p[f"e{e}.up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ p[f"e{e}.down"].T


def sparse_ff(h, p, ml):
    idx, wts = route(h, p, ml["router"])
    limit = float(ml["expert"]["limit"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(idx.shape[1]):
            out[t] += expert_ff(wts[t, k] * h[t:t + 1], p, int(idx[t, k]), limit)[0]
    return out


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


MIXERS = {"attention": sink_attention_mixer, "parallel": parallel_mixer}


def layer_runs(config):
    """[(layer index, pass number or None)] in execution order; the pass number is set on a pass's first layer"""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def forward(config, weights, tokens, dtype=torch.float64, collect=None):
    """Logits [T, vocab] of one sequence; `collect` (a list) receives the residual stream after every layer run."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    e = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = e
    for i, t in layer_runs(config):
        if t is not None:
            x = x + w["loop.step"][t] + (e if t > 0 else 0)
        spec, p = config["layers"][i], sub(w, f"l{i}.")
        x = x + MIXERS[spec["type"]](rms_norm(x, p["norm1"], eps), sub(p, "mix."), spec["mixer"], eps)
        ml = spec.get("mlp")
        if ml is not None:
            x = x + sparse_ff(rms_norm(x, p["norm2"], eps), sub(p, "mlp."), ml)
        if collect is not None:
            collect.append(x)
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T


def tensor_shapes(config):
    """name -> shape of a checkpoint of this configuration"""
    W, V = int(config["width"]), int(config["vocab"])
    out = {"embed": (V, W), "final.norm": (W,)}
    if config.get("loop"):
        out["loop.step"] = (int(config["loop"]["times"]), W)

    def attn(pre, m, sink):
        H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        out.update({pre + "q": (H * D, W), pre + "k": (G * D, W), pre + "v": (G * Dv, W), pre + "o": (W, H * Dv)})
        if sink:
            out[pre + "sink"] = (H,)
        else:
            out[pre + "talk"] = (H, H)
            if m.get("conv"):
                taps = int(m["conv"])
                out.update({pre + "q.conv": (H * D, taps), pre + "k.conv": (G * D, taps), pre + "v.conv": (G * Dv, taps)})

    for i, spec in enumerate(config["layers"]):
        pre, m = f"l{i}.", spec["mixer"]
        out[pre + "norm1"] = (W,)
        if spec["type"] == "attention":
            attn(pre + "mix.", m, True)
        elif spec["type"] == "parallel":
            attn(pre + "mix.left.", m["left"], False)
            r = m["right"]
            H, D, Dv = int(r["heads"]), int(r["dim"]), int(r["vdim"])
            out.update({pre + "mix.right.q": (H * D, W), pre + "mix.right.k": (H * D, W), pre + "mix.right.v": (H * Dv, W),
                        pre + "mix.right.g": (H * Dv, W), pre + "mix.right.o": (W, H * Dv)})
        else:
            raise ValueError(spec["type"])
        ml = spec.get("mlp")
        if ml is None:
            continue
        F, E = int(ml["expert"]["ff"]), int(ml["router"]["experts"])
        out.update({pre + "norm2": (W,), pre + "mlp.router": (E, W)})
        for e in range(E):
            out.update({pre + f"mlp.e{e}.gate": (F, W), pre + f"mlp.e{e}.up": (F, W), pre + f"mlp.e{e}.down": (W, F)})
    return out


def random_model(config, seed=0, overrides=None):
    """Random bf16-representable weights (so that a bf16 checkpoint of them is exact) under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        leaf = name.rsplit(".", 1)[-1]
        if "norm" in leaf:
            t = torch.randn(shape, generator=g) * 0.1
        elif leaf == "sink":
            t = torch.randn(shape, generator=g)
        elif leaf == "talk":
            t = torch.eye(shape[0]) + torch.randn(shape, generator=g) * 0.3
        elif leaf == "conv":
            t = torch.randn(shape, generator=g) * 0.5
        elif name == "loop.step":
            t = torch.randn(shape, generator=g) * 0.1
        elif name == "embed":
            t = torch.randn(shape, generator=g) * 0.5
        elif leaf in ("down", "o"):    # sublayer outputs well below the stream: an expert swapped at a router's near-tie
            t = torch.randn(shape, generator=g) * ((0.15 if leaf == "down" else 0.4) * shape[-1] ** -0.5)   # (bf16 serving)
        else:
            t = torch.randn(shape, generator=g) * (1.5 * shape[-1] ** -0.5)
        out[name] = t.to(torch.bfloat16).to(torch.float32)
    for k, v in (overrides or {}).items():
        out[k] = v.to(torch.bfloat16).to(torch.float32)
    return out

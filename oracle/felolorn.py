"""Plain, slow statement of the Felolorn design (torch on CPU, float64 by default): one function per mechanism.

TEST INFRASTRUCTURE: nothing of the product path imports this file and it imports nothing of the product path.
One sequence at a time, whole, with dense [T, T] score matrices and Python loops over time for the recurrences.

Notation (W x means `x @ W.T`, weights stored [out, in]; t = position, counted from 0):

  norm          n(x; w) = x / sqrt(mean(x^2) + eps) * w
  layer         h = n(x; w_1);   g = sigmoid(W_rg1 h + b_rg1);   u = h + conv(h)
                x <- x + n(g * mixer(u); w_1b)
                h = n(x; w_2);   g = sigmoid(W_rg2 h + b_rg2)
                x <- x + n(g * ff(h); w_2b)                                  (a layer may have no feed-forward)
  conv          conv(h)_t[c] = sum_{j < taps} w[c, j] * h_{t - (taps - 1) + j}[c],  h before position 0 is zero
  latent attn   c_q = n(W_dq u; w_dq),  q = W_uq c_q;   c = n(W_dkv u; w_dkv);   k_h = W_uk,h c,  v_h = W_uv,h c
                s_ij = scale * q_i . k_j  (j <= i);   p_ij = exp(s_ij) / (exp(sink_h) + sum_j' exp(s_ij'))
                out = W_o concat_h(sum_j p_ij v_j)
  lightning     q = silu(W_q u), k = silu(W_k u), v = silu(W_v u);  per head  S_t = decay_h S_{t-1} + k_t v_t^T,  o_t = S_t^T q_t
                out = W_o (n(concat_h(o); w) * sigmoid(W_g u))
  hgrn2         q = silu(W_q u), v = W_v u,  f = l + (1 - l) * sigmoid(W_f u + b_f)    (l: a lower bound per channel)
                per head  S_t = diag(f_t) S_{t-1} + (1 - f_t) v_t^T,  o_t = S_t^T q_t;   out = W_o concat_h(n(o_h; w))
  sparse ff     s = sigmoid(W_r h);  choice = s + correction;  groups of neighbouring experts, a group's value = the sum
                of its two largest choice values;  only the best `keep` groups stay eligible;  the `top` largest choice
                values among them are taken;  out = sum_k s_k W_d,k (silu(W_g,k h) * (W_u,k h))
  output        z = E n(x; w_final)  (E: the embedding table, unscaled);  logits = cap * tanh(z / cap)
  embedding     x = E[token] * embedding scale
"""
from __future__ import annotations

import torch


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def input_conv(h, w):
    """h [T, C], w [C, taps] -> conv(h) [T, C] (without the h it is added to)"""
    T, taps = h.shape[0], w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, h.shape[1], dtype=h.dtype), h])
    out = torch.zeros_like(h)
    for j in range(taps):
        out = out + w[:, j] * padded[j:j + T]
    return out


def latent_attention_mixer(u, p, m, eps):
    T = u.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    cq = rms_norm(u @ p["dq"].T, p["dq.norm"], eps)
    q = (cq @ p["uq"].T).view(T, H, D)
    c = rms_norm(u @ p["dkv"].T, p["dkv.norm"], eps)
    k = (c @ p["uk"].T).view(T, H, D)
    v = (c @ p["uv"].T).view(T, H, Dv)
    s = torch.einsum("ihd,jhd->hij", q, k) * float(m["scale"])
    hidden = torch.arange(T).view(1, T) > torch.arange(T).view(T, 1)
    s = s.masked_fill(hidden, float("-inf"))
    sink = p["sink"].view(H, 1, 1).expand(H, T, 1)
    pr = torch.softmax(torch.cat([s, sink], -1), -1)[..., :T]     # the sink takes weight and gives nothing
    o = torch.einsum("hij,jhd->ihd", pr, v).reshape(T, H * Dv)
    return o @ p["o"].T


def lightning_mixer(u, p, m, eps):
    T = u.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    decay = torch.tensor([float(d) for d in m["decay"]], dtype=u.dtype)
    q = silu(u @ p["q"].T).view(T, H, D)
    k = silu(u @ p["k"].T).view(T, H, D)
    v = silu(u @ p["v"].T).view(T, H, Dv)
    S = torch.zeros(H, D, Dv, dtype=u.dtype)
    out = []
    for t in range(T):
        S = decay.view(H, 1, 1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out.append(torch.einsum("hdv,hd->hv", S, q[t]).reshape(H * Dv))
    o = rms_norm(torch.stack(out), p["norm"], eps) * torch.sigmoid(u @ p["g"].T)
    return o @ p["o"].T


def hgrn2_mixer(u, p, m, eps):
    T = u.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(u @ p["q"].T).view(T, H, D)
    v = (u @ p["v"].T).view(T, H, Dv)
    low = p["lower"]
    f = (low + (1 - low) * torch.sigmoid(u @ p["f"].T + p["f.b"])).view(T, H, D)
    S = torch.zeros(H, D, Dv, dtype=u.dtype)
    out = []
    for t in range(T):
        S = f[t].unsqueeze(-1) * S + (1 - f[t]).unsqueeze(-1) * v[t].unsqueeze(-2)
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    o = rms_norm(torch.stack(out), p["norm"], eps).reshape(T, H * Dv)   # per head, over the value channels
    return o @ p["o"].T


def route(h, p, r):
    """-> (chosen experts [T, top], their weights [T, top])"""
    E, top = int(r["experts"]), int(r["top"])
    g = r.get("groups") or {"count": 1, "keep": 1}
    count, keep = int(g["count"]), int(g["keep"])
    s = torch.sigmoid(h @ p["router"].T)
    choice = s + p["correction"]
    per = E // count
    grouped = choice.view(-1, count, per)
    value = torch.topk(grouped, min(2, per), dim=-1).values.sum(-1)          # [T, count]
    eligible = torch.zeros_like(value, dtype=torch.bool)
    eligible.scatter_(1, torch.topk(value, keep, dim=-1).indices, True)
    masked = grouped.masked_fill(~eligible.unsqueeze(-1), float("-inf")).reshape(-1, E)
    idx = torch.topk(masked, top, dim=-1).indices
    return idx, torch.gather(s, 1, idx)


def expert_ff(h, p, e):
    return (silu(h @ p[f"e{e}.gate"].T) * (h @ p[f"e{e}.up"].T)) @ p[f"e{e}.down"].T


def sparse_ff(h, p, ml):
    idx, wts = route(h, p, ml["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(idx.shape[1]):
            out[t] += wts[t, k] * expert_ff(h[t:t + 1], p, int(idx[t, k]))[0]
    return out


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


MIXERS = {"latent_attention": latent_attention_mixer, "lightning": lightning_mixer, "hgrn2": hgrn2_mixer}


def forward(config, weights, tokens, dtype=torch.float64, collect=None):
    """Logits [T, vocab] of one sequence; `collect` (a list) receives the residual stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float((config.get("embedding") or {}).get("scale", 1.0))
    for i, spec in enumerate(config["layers"]):
        p = sub(w, f"l{i}.")
        h = rms_norm(x, p["norm1"], eps)
        g = torch.sigmoid(h @ p["rg1"].T + p["rg1.b"])
        u = h + input_conv(h, p["canon1"])
        y = MIXERS[spec["type"]](u, sub(p, "mix."), spec["mixer"], eps)
        x = x + rms_norm(g * y, p["norm1b"], eps)
        ml = spec.get("mlp")
        if ml is not None:
            h = rms_norm(x, p["norm2"], eps)
            g = torch.sigmoid(h @ p["rg2"].T + p["rg2.b"])
            x = x + rms_norm(g * sparse_ff(h, sub(p, "mlp."), ml), p["norm2b"], eps)
        if collect is not None:
            collect.append(x)
    z = rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    cap = float(config.get("logit_softcap") or 0.0)
    return cap * torch.tanh(z / cap) if cap > 0 else z


def tensor_shapes(config):
    """name -> shape of a checkpoint of this configuration"""
    W, V = int(config["width"]), int(config["vocab"])
    taps = int(config["canon"]["taps"])
    out = {"embed": (V, W), "final.norm": (W,)}
    for i, spec in enumerate(config["layers"]):
        pre, m = f"l{i}.", spec["mixer"]
        H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        out.update({pre + "norm1": (W,), pre + "norm1b": (W,), pre + "canon1": (W, taps), pre + "rg1": (W, W),
                    pre + "rg1.b": (W,)})
        if spec["type"] == "latent_attention":
            C, Q = int(m["kv_rank"]), int(m["q_rank"])
            out.update({pre + "mix.dq": (Q, W), pre + "mix.dq.norm": (Q,), pre + "mix.uq": (H * D, Q),
                        pre + "mix.dkv": (C, W), pre + "mix.dkv.norm": (C,), pre + "mix.uk": (H * D, C),
                        pre + "mix.uv": (H * Dv, C), pre + "mix.sink": (H,), pre + "mix.o": (W, H * Dv)})
        elif spec["type"] == "lightning":
            out.update({pre + "mix.q": (H * D, W), pre + "mix.k": (H * D, W), pre + "mix.v": (H * Dv, W),
                        pre + "mix.g": (H * Dv, W), pre + "mix.norm": (H * Dv,), pre + "mix.o": (W, H * Dv)})
        elif spec["type"] == "hgrn2":
            out.update({pre + "mix.q": (H * D, W), pre + "mix.f": (H * D, W), pre + "mix.f.b": (H * D,),
                        pre + "mix.lower": (H * D,), pre + "mix.v": (H * Dv, W), pre + "mix.norm": (Dv,),
                        pre + "mix.o": (W, H * Dv)})
        else:
            raise ValueError(spec["type"])
        ml = spec.get("mlp")
        if ml is None:
            continue
        F, E = int(ml["expert"]["ff"]), int(ml["router"]["experts"])
        out.update({pre + "norm2": (W,), pre + "norm2b": (W,), pre + "rg2": (W, W), pre + "rg2.b": (W,),
                    pre + "mlp.router": (E, W), pre + "mlp.correction": (E,)})
        for e in range(E):
            out.update({pre + f"mlp.e{e}.gate": (F, W), pre + f"mlp.e{e}.up": (F, W), pre + f"mlp.e{e}.down": (W, F)})
    return out


def random_model(config, seed=0, overrides=None):
    """Random bf16-representable weights (so that a bf16 checkpoint of them is exact) under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        leaf = name.split(".", 1)[-1] if name.startswith("l") else name
        if "norm" in leaf:
            t = 1 + torch.randn(shape, generator=g) * 0.1
        elif leaf == "mix.lower":
            t = torch.rand(shape, generator=g) * 0.9
        elif leaf == "mix.sink":
            t = torch.randn(shape, generator=g)
        elif leaf == "mlp.correction":
            t = torch.randn(shape, generator=g) * 0.2
        elif leaf.endswith(".b"):
            t = torch.randn(shape, generator=g) * 0.5
        elif leaf == "canon1":
            t = torch.randn(shape, generator=g) * 0.3
        elif name == "embed":
            t = torch.randn(shape, generator=g) * 0.1
        else:
            t = torch.randn(shape, generator=g) * (1.5 * shape[-1] ** -0.5)
        out[name] = t.to(torch.bfloat16).to(torch.float32)
    for k, v in (overrides or {}).items():
        out[k] = v.to(torch.bfloat16).to(torch.float32)
    return out

"""Plain, slow float64 restatement of the Gupuvik design, one function per mechanism, for the tests only.

Nothing here is shared with the product path: it reads the configuration dictionary itself, recomputes whole sequences from
their first token (no cache, no carried state: the recurrence simply runs over all tokens), loops over heads, tokens and
experts.  Weights are dicts of float64 torch tensors under the checkpoint's names.

A layer is PARALLEL: one norm, then  x <- x + a1 * mixer(h) + a2 * ff(h)  with  h = norm1(x)  and  a_i = sigmoid(R_i h + r_i)
(element-wise gates of the two sublayers).  The norm has a single learned number as its gain.
"""
import math

import torch

F = torch.float64


# ------------------------------------------------------------------------------------------------ small pieces
def scalar_rms_norm(x, gain, eps):
    """x / sqrt(mean(x^2) + eps) * gain, one gain for all coordinates."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def visible(i, j, size, keep_first):
    """May position i look at position j under a sliding window that also keeps the sequence's first tokens?"""
    return j <= i and (i - j < size or j < keep_first)


def causal_conv_silu(x, taps):
    """x [T, C], taps [C, n]: y[t] = silu(sum_s taps[:, n - 1 - s] * x[t - s]) with zeros before the first token."""
    T, n = x.shape[0], taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for s in range(n):
            if t - s >= 0:
                y[t] += taps[:, n - 1 - s] * x[t - s]
    return silu(y)


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


# ------------------------------------------------------------------------------------------------ mixers
def attention_keys_values(h, w, pre):
    """Keys and values of a layer that owns its projections: [T, G * dim], [T, G * vdim]."""
    return h @ w[pre + "k"].T + w[pre + "k.b"], h @ w[pre + "v"].T + w[pre + "v.b"]


def capped_window_attention(h, w, pre, m, keys, values):
    """h [T, W] of one sequence from its first token; keys / values [T, G * dim] / [T, G * vdim] (the layer's own or another's)."""
    T, H, G, D, V = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).view(T, H, D)
    k, v = keys.view(T, G, D), values.view(T, G, V)
    mask = m.get("mask") or {}
    size, keep = mask.get("size", T + 1), mask.get("keep_first", 0)
    cap = m.get("softcap")
    gate = torch.sigmoid(h @ w[pre + "g"].T)                                   # [T, H]
    allowed = torch.tensor([[visible(i, j, size, keep) for j in range(T)] for i in range(T)])
    out = torch.zeros(T, H, V, dtype=F)
    for hd in range(H):
        kv = hd // (H // G)
        s = (q[:, hd] @ k[:, kv].T) * m["scale"] * w[pre + "temp"][hd]
        if cap:
            s = cap * torch.tanh(s / cap)
        p = torch.softmax(s.masked_fill(~allowed, -math.inf), -1)
        out[:, hd] = (p @ v[:, kv]) * gate[:, hd, None]
    return out.reshape(T, H * V) @ w[pre + "o"].T


def delta_rule_inputs(h, w, pre, m):
    """Everything the recurrence consumes: q, k [T, Hk, dim] (unit vectors, q scaled), v [T, H, vdim], beta [T, H],
    decay [T, H, dim]."""
    T, H, Hk, D, V = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit(causal_conv_silu(h @ w[pre + "q"].T, w[pre + "q.conv"]).view(T, Hk, D)) * D ** -0.5
    k = unit(causal_conv_silu(h @ w[pre + "k"].T, w[pre + "k.conv"]).view(T, Hk, D))
    v = causal_conv_silu(h @ w[pre + "v"].T, w[pre + "v.conv"]).view(T, H, V)
    beta = torch.sigmoid(h @ w[pre + "b"].T)
    dt = softplus((h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(w[pre + "A_log"])[None, :, None] * dt)
    return q, k, v, beta, decay


def delta_rule_scan(q, k, v, beta, decay):
    """Per head, a matrix memory S [dim, vdim] from zero:  S <- diag(decay) S;  u = beta (v - S^T k);  S <- S + k u^T;
    o = S^T q (the read-out sees the write of its own token)."""
    T, H, V = v.shape
    Hk, D = k.shape[1], k.shape[2]
    o = torch.zeros(T, H, V, dtype=F)
    for hd in range(H):
        kh = hd // (H // Hk)
        S = torch.zeros(D, V, dtype=F)
        for t in range(T):
            S = decay[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            o[t, hd] = S.T @ q[t, kh]
    return o


def channel_delta(h, w, pre, m, eps):
    T, H, V = h.shape[0], m["heads"], m["vdim"]
    o = delta_rule_scan(*delta_rule_inputs(h, w, pre, m))
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w[pre + "norm"]
    o = o * torch.sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T).view(T, H, V)
    return o.reshape(T, H * V) @ w[pre + "o"].T


# ------------------------------------------------------------------------------------------------ feed-forward
def dense_ff(h, w, pre):
    return gelu_tanh(h @ w[pre + "up"].T) @ w[pre + "down"].T


def route(h, w, pre, top):
    """Chosen experts [T, top] and their weights: softmax over the chosen logits only."""
    z = h @ w[pre + "router"].T
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, -1), z


def moe_ff(h, w, pre, ff):
    idx, wt, _ = route(h, w, pre, ff["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for s in range(idx.shape[1]):
            e = pre + f"e{int(idx[t, s])}."
            out[t] += wt[t, s] * ((silu(h[t] @ w[e + "gate"].T) * (h[t] @ w[e + "up"].T)) @ w[e + "down"].T)
    return out


# ------------------------------------------------------------------------------------------------ the model
def forward(tokens, w, cfg, return_layers=False):
    """Logits [T, vocab] of one sequence given from its first token (and the residual stream after every layer)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    kv, trace = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = scalar_rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kv[i] = attention_keys_values(h, w, p + "mix.")
                src = i
            y = capped_window_attention(h, w, p + "mix.", m, *kv[src])
        elif layer["type"] == "channel_delta":
            y = channel_delta(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        upd = torch.sigmoid(h @ w[p + "rg1"].T + w[p + "rg1.b"]) * y
        ff = layer.get("mlp")
        if ff is not None:
            f = dense_ff(h, w, p + "mlp.") if ff["kind"] == "dense" else moe_ff(h, w, p + "mlp.", ff)
            upd = upd + torch.sigmoid(h @ w[p + "rg2"].T + w[p + "rg2.b"]) * f
        x = x + upd
        trace.append(x.clone())
    logits = scalar_rms_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(trace)) if return_layers else logits


def min_router_margin(tokens, w, cfg):
    """Smallest relative gap between the last chosen and the first rejected router logit over all tokens and layers (a gap near
    zero means a bf16 run may legitimately pick another expert)."""
    eps = cfg["norm"]["eps"]
    _, trace = forward(tokens, w, cfg, return_layers=True)
    x = w["embed"][torch.tensor(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    worst = math.inf
    for i, layer in enumerate(cfg["layers"]):
        ff = layer.get("mlp")
        if ff is not None and ff["kind"] == "moe" and ff["router"]["top"] < ff["router"]["experts"]:
            h = scalar_rms_norm(x, w[f"l{i}.norm1"], eps)
            z = torch.sort(h @ w[f"l{i}.mlp.router"].T, -1, descending=True).values
            k = ff["router"]["top"]
            worst = min(worst, float(((z[:, k - 1] - z[:, k]) / z.abs().max(-1).values.clamp_min(1e-9)).min()))
        x = trace[i]
    return worst

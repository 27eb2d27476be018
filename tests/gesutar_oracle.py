"""Plain, slow float64 restatement of the Gesutar design, one function per mechanism, for the tests only.

Nothing here is shared with the product path: keys and values are expanded per head (the product works in the latent space),
whole sequences are recomputed from scratch (the product reads a paged cache), experts are looped token by token.
Notation: T tokens, W width, H heads, per head `dim` unrotated + `rd` rotated query/key dimensions, `vd` value dimensions,
latent size R.  Weights are dicts of float64 torch tensors under the checkpoint's names.
"""
import math

import torch

F = torch.float64


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def hashed_bigram_rows(tokens, first_prev, buckets, mul_prev, mul_cur):
    """Row of the bigram table for each token; the row past the buckets stands for "no previous token"."""
    rows, prev = [], first_prev
    for t in tokens:
        rows.append(buckets if prev < 0 else (prev * mul_prev + t * mul_cur) % buckets)
        prev = t
    return rows


def embed(tokens, weights, spec, first_prev=-1):
    x = weights["embed"][torch.tensor(tokens)] * spec.embed_scale
    if spec.bigram_buckets:
        rows = hashed_bigram_rows(tokens, first_prev, spec.bigram_buckets, spec.bigram_mul_prev, spec.bigram_mul_cur)
        x = x + weights["bigram"][torch.tensor(rows)]
    return x


def rotate_pairs(x, positions, dims, base):
    """Rotate the pairs (2i, 2i + 1), i < dims / 2, of the last axis by positions * base^(-2i / dims); the rest passes."""
    out = x.clone()
    for i in range(dims // 2):
        ang = positions.to(F) * base ** (-2.0 * i / dims)
        c, s = torch.cos(ang), torch.sin(ang)
        while c.dim() < x.dim() - 1:
            c, s = c.unsqueeze(-1), s.unsqueeze(-1)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def softmax_with_sink(scores, allowed, sink):
    """Softmax over the allowed keys whose denominator also counts exp(sink) once (sink None: plain softmax)."""
    s = scores.masked_fill(~allowed, -math.inf)
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink)
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink - m)
    return e / den


def latent_attention(h, positions, w, pre, l, eps):
    """h [T, W] -> mixer output [T, W] for one sequence given from its first token."""
    T, H = h.shape[0], l.heads
    q = (h @ w[pre + "q"].T).view(T, H, l.dim + l.rot_dim)
    down = h @ w[pre + "dkv"].T
    c = rms_norm(down[:, :l.kv_rank], w[pre + "dkv.norm"], eps)
    k_shared = rotate_pairs(down[:, l.kv_rank:], positions, l.rot_dims, l.rot_base)            # [T, rd]
    k_plain = (c @ w[pre + "uk"].T).view(T, H, l.dim)
    val = (c @ w[pre + "uv"].T).view(T, H, l.vdim)
    q_plain, q_rot = q[..., :l.dim], rotate_pairs(q[..., l.dim:], positions, l.rot_dims, l.rot_base)
    out = torch.zeros(T, H, l.vdim, dtype=F)
    gap = positions[:, None] - positions[None, :]
    allowed = (gap >= 0) & (gap < l.window)
    for hd in range(H):
        sc = (q_plain[:, hd] @ k_plain[:, hd].T + q_rot[:, hd] @ k_shared.T) * l.scale
        p = softmax_with_sink(sc, allowed, w[pre + "sink"][hd])
        out[:, hd] = p @ val[:, hd]
    gate = torch.sigmoid(h @ w[pre + "g"].T)
    return (out.reshape(T, H * l.vdim) * gate) @ w[pre + "o"].T


def grouped_router(z, experts, groups, keep, top, scale):
    """z [T, E] logits -> (ids [T, top], weights [T, top])."""
    p = torch.softmax(z.to(F), -1)
    ids, wts = [], []
    size = experts // groups
    for row in p:
        best = sorted(range(groups), key=lambda g: (-float(row[g * size:(g + 1) * size].max()), g))[:keep]
        cand = [e for g in best for e in range(g * size, (g + 1) * size)]
        chosen = sorted(cand, key=lambda e: (-float(row[e]), e))[:top]
        sel = row[torch.tensor(chosen)]
        ids.append(chosen)
        wts.append(sel / (sel.sum() + 1e-20) * scale)
    return ids, torch.stack(wts)


def router_margin(z, experts, groups, keep, top):
    """Smallest relative gap, over the rows of z, between what the router keeps and what it drops (last kept group against first
    dropped group, last chosen expert against first dropped candidate).  A test in reduced precision is only meaningful on
    inputs whose margin is well above that precision's rounding."""
    p = torch.softmax(z.to(F), -1)
    size, worst = experts // groups, 1.0
    for row in p:
        gs = sorted((float(row[g * size:(g + 1) * size].max()) for g in range(groups)), reverse=True)
        if keep < groups:
            worst = min(worst, (gs[keep - 1] - gs[keep]) / gs[keep - 1])
        best = sorted(range(groups), key=lambda g: (-float(row[g * size:(g + 1) * size].max()), g))[:keep]
        cand = sorted((float(row[e]) for g in best for e in range(g * size, (g + 1) * size)), reverse=True)
        if top < len(cand):
            worst = min(worst, (cand[top - 1] - cand[top]) / cand[top - 1])
    return worst


def squared_relu_ff(h, up, down):
    return (torch.relu(h @ up.T) ** 2) @ down.T


def moe(h, w, pre, l):
    ids, wts = grouped_router(h @ w[pre + "router"].T, l.experts, l.groups, l.keep_groups, l.top, l.router_scale)
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j, e in enumerate(ids[t]):
            y[t] += wts[t, j] * squared_relu_ff(h[t], w[pre + f"e{e}.up"], w[pre + f"e{e}.down"])
    if l.shared_ff:
        y = y + squared_relu_ff(h, w[pre + "shared.up"], w[pre + "shared.down"])
    return y


def forward(spec, weights, tokens, return_layers=False, margins=None):
    """Logits [T, vocab] of one sequence from its first token (float64), and the residual stream after every layer.
    margins: a list that receives every layer's router_margin."""
    w = {k: v.to(F) for k, v in weights.items()}
    x = embed(tokens, w, spec)
    positions = torch.arange(len(tokens))
    layers = []
    for i, l in enumerate(spec.layers):
        x = x + latent_attention(rms_norm(x, w[f"l{i}.norm1"], spec.norm_eps), positions, w, f"l{i}.mix.", l, spec.norm_eps)
        if l.mlp:
            h2 = rms_norm(x, w[f"l{i}.norm2"], spec.norm_eps)
            if margins is not None:
                margins.append(router_margin(h2 @ w[f"l{i}.mlp.router"].T, l.experts, l.groups, l.keep_groups, l.top))
            x = x + moe(h2, w, f"l{i}.mlp.", l)
        layers.append(x.clone())
    logits = rms_norm(x, w["final.norm"], spec.norm_eps) @ w["head"].T
    return (logits, layers) if return_layers else logits


def greedy(spec, weights, prompt, new_tokens):
    seq, out = list(prompt), []
    for _ in range(new_tokens):
        nxt = int(torch.argmax(forward(spec, weights, seq)[-1]))
        out.append(nxt)
        seq.append(nxt)
    return out

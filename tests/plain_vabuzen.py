"""Vabuzen in plain float64 PyTorch, one function per mechanism, whole sequences at a time.

Nothing here is shared with the library: the functions take the dictionary of config.json and
a dictionary of tensors by checkpoint name, and run one request's tokens from position 0.
Slow on purpose: loops over tokens, heads and keys where the definition has them.

The model: token embedding; layers `x += m * post(sublayer(pre(x)))` for a mixer and a
feed-forward, every norm a "dynamic tanh" (no statistics: `tanh(alpha x) w + b`); two kinds of
mixer (grouped-query attention behind short convolutions, inside a sliding window that also keeps
the sequence's first tokens, with one added to the softmax's denominator; attention over a
compressed row shared by all heads); dense or routed feed-forwards (experts chosen inside the best
groups, plus one expert every token uses); a range of layers that runs several times, before every
run of which a vector of that run (and, from the second run on, the embedding's rows) is added;
final norm, head, and logits bent by `cap tanh(z / cap)`.
"""
import json
import math
import os

import torch
from safetensors.torch import load_file

F64 = torch.float64


def load_model_folder(folder):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    return cfg, {k: v.to(F64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


# ------------------------------------------------------------------ small pieces
def dynamic_tanh(x, W, name):
    return torch.tanh(W[name + ".alpha"] * x) * W[name] + W[name + ".b"]


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def causal_taps(u, w):
    """u [n, channels], w [channels, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before 0."""
    n, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def turn(u, v, angle):
    c, s = torch.cos(angle), torch.sin(angle)
    return u * c - v * s, v * c + u * s


def rotate_neighbours(x, positions, base, dims):
    """x [n, heads, size]: values 2i and 2i+1 form pair i (i < dims/2); the rest passes."""
    out = x.clone()
    for i in range(dims // 2):
        angle = (positions.to(F64) * float(base) ** (-2.0 * i / dims))[:, None]
        out[..., 2 * i], out[..., 2 * i + 1] = turn(x[..., 2 * i], x[..., 2 * i + 1], angle)
    return out


def rotate_halves(x, positions, base, dims):
    """x [n, heads, size]: values i and i + dims/2 form pair i (i < dims/2); the rest passes."""
    out, half = x.clone(), dims // 2
    for i in range(half):
        angle = (positions.to(F64) * float(base) ** (-2.0 * i / dims))[:, None]
        out[..., i], out[..., i + half] = turn(x[..., i], x[..., i + half], angle)
    return out


# ------------------------------------------------------------------ mixers
def window_attention(h, W, p, m):
    """Grouped queries, a convolution per channel behind each of the three projections, neighbouring
    pairs turned, keys of the last `size` positions and of the first `keep_first` ones, and a
    softmax whose denominator holds a one more."""
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ W[p + "q"].T, h @ W[p + "k"].T, h @ W[p + "v"].T
    if m.get("conv"):
        q, k, v = causal_taps(q, W[p + "q.conv"]), causal_taps(k, W[p + "k.conv"]), causal_taps(v, W[p + "v.conv"])
    q, k, v = q.view(n, H, D), k.view(n, G, D), v.view(n, G, Dv)
    pos = torch.arange(n)
    rot = m.get("rot")
    if rot and rot["dims"]:
        q, k = rotate_neighbours(q, pos, rot["base"], rot["dims"]), rotate_neighbours(k, pos, rot["base"], rot["dims"])
    mask = m.get("mask") or {}
    size, keep = mask.get("size"), mask.get("keep_first", 0)
    out = torch.zeros(n, H, Dv, dtype=F64)
    for i in range(n):
        seen = [j for j in range(i + 1) if size is None or i - j < size or j < keep]
        for a in range(H):
            g = a // (H // G)
            s = (k[seen, g] @ q[i, a]) * m["scale"]
            top = max(float(s.max()), 0.0)
            e = torch.exp(s - top)
            out[i, a] = (e / (math.exp(-top) + e.sum())) @ v[seen, g]
    return out.reshape(n, H * Dv) @ W[p + "o"].T


def compressed_attention(h, W, p, m, eps):
    """Every head's keys and values come from one normed row c of `kv_rank` numbers per token; a
    turned key part of `rot_dim` numbers is shared by all heads.  Ordinary causal softmax."""
    n = h.shape[0]
    H, D, R, Dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ W[p + "q"].T).view(n, H, D + R)
    down = h @ W[p + "dkv"].T
    c = unit_rms(down[:, :rank], eps) * W[p + "dkv.norm"]
    pos = torch.arange(n)
    base = m["rot"]["base"] if R else 1.0
    q_turn = rotate_halves(q[..., D:], pos, base, R)
    k_turn = rotate_halves(down[:, None, rank:], pos, base, R)[:, 0]
    k_plain, v = (c @ W[p + "uk"].T).view(n, H, D), (c @ W[p + "uv"].T).view(n, H, Dv)
    out = torch.zeros(n, H, Dv, dtype=F64)
    for i in range(n):
        for a in range(H):
            s = (k_plain[: i + 1, a] @ q[i, a, :D] + k_turn[: i + 1] @ q_turn[i, a]) * m["scale"]
            out[i, a] = torch.softmax(s, 0) @ v[: i + 1, a]
    return out.reshape(n, H * Dv) @ W[p + "o"].T


# ------------------------------------------------------------------ feed-forwards
def dense_ff(h, W, p):
    return gelu_tanh(h @ W[p + "up"].T + W[p + "up.b"]) @ W[p + "down"].T + W[p + "down.b"]


def gated_expert(x, W, p):
    return W[p + "down"] @ (silu(W[p + "gate"] @ x) * (W[p + "up"] @ x))


def choose_experts(score, r):
    """score [experts] -> (chosen experts, their weights).  Only the `keep` groups whose two largest
    scores add up to most can give experts; the weights are the chosen scores over their sum, times
    the router's scale."""
    E, top = r["experts"], r["top"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    per = E // groups["count"]
    def group_score(g):
        return float(sum(sorted((float(score[e]) for e in range(g * per, (g + 1) * per)), reverse=True)[:2]))
    best = sorted(range(groups["count"]), key=lambda g: (-group_score(g), g))[: groups["keep"]]
    allowed = [e for e in range(E) if e // per in best]
    chosen = sorted(allowed, key=lambda e: (-float(score[e]), e))[:top]
    total = sum(score[e] for e in chosen) + 1e-20
    return chosen, [score[e] / total * r.get("scale", 1.0) for e in chosen]


def routed_ff(h, W, p, f):
    score = torch.sigmoid(h @ W[p + "router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen, weights = choose_experts(score[t], f["router"])
        for e, w in zip(chosen, weights):
            out[t] += w * gated_expert(h[t], W, f"{p}e{e}.")
        if f.get("shared"):
            out[t] += gated_expert(h[t], W, p + "shared.")
    return out


# ------------------------------------------------------------------ the model
def run_order(cfg):
    """[(layer, number of the run if this entry is the first of a run of the looped range)]."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def model_hidden(cfg, W, tokens):
    """The residual stream after every entry of the run order: list of [n, width]."""
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x0 = W["embed"][torch.tensor(tokens)]
    x, after = x0.clone(), []
    for L, run in run_order(cfg):
        if run is not None:
            if run > 0:
                x = x + x0
            x = x + W["loop.step"][run]
        layer, p = cfg["layers"][L], f"l{L}."
        h = dynamic_tanh(x, W, p + "norm1")
        if layer["type"] == "attention":
            y = window_attention(h, W, p + "mix.", layer["mixer"])
        else:
            y = compressed_attention(h, W, p + "mix.", layer["mixer"], eps)
        x = x + mult * dynamic_tanh(y, W, p + "norm1b")
        f = layer.get("mlp")
        if f:
            h = dynamic_tanh(x, W, p + "norm2")
            y = dense_ff(h, W, p + "mlp.") if f["kind"] == "dense" else routed_ff(h, W, p + "mlp.", f)
            x = x + mult * dynamic_tanh(y, W, p + "norm2b")
        after.append(x)
    return after


def model_logits(cfg, W, tokens):
    z = dynamic_tanh(model_hidden(cfg, W, tokens)[-1], W, "final.norm") @ W["head"].T
    cap = cfg.get("logit_softcap")
    return (cap * torch.tanh(z / cap) if cap else z).to(torch.float32)


def greedy(cfg, W, prompt, n_new):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(model_logits(cfg, W, tokens)[-1].argmax()))
    return tokens[len(prompt):]

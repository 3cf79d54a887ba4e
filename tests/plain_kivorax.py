"""Kivorax in plain float64 PyTorch, one function per mechanism, whole sequences at a time.

Nothing here is shared with the library: the functions take a configuration (the dictionary
of config.json) and a dictionary of tensors by checkpoint name, and run one request's
tokens from position 0.  Slow on purpose: loops over tokens, heads and experts where the
definition has them.

The model: token embedding times a constant; layers `x += mixer(n(x)) + ff(n(x))` with one
RMS norm n for both sub-layers; behind them a gated row of a per-layer token table, normed,
is added; what a layer hands on is a weighted sum of the embedding's rows and the results of
all layers so far; final RMS norm; a head matrix of its own.  Mixers: a pair (softmax
attention with a logarithmic distance bias beside a gated linear recurrent unit, the mean of
their normed outputs), a delta rule with a decay per key channel, gated linear attention.
Feed-forwards: dense with biases and gelu, or routed experts with squared relu.
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


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.logaddexp(z, torch.zeros_like(z))


def causal_conv(x, taps, bias=None):
    """x [T, C], taps [C, K] (the last column is the current token's), zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(K):
            src = t - (K - 1 - j)
            if src >= 0:
                out[t] += taps[:, j] * x[src]
    return out if bias is None else out + bias


# ------------------------------------------------------------------ the pair's left side
def query_factor(position, q_temp):
    if not q_temp:
        return 1.0
    return 1.0 + q_temp["coef"] * math.log((position + 1) // q_temp["every"] + 1)


def distance_bias_attention(h, m, t, p):
    """Grouped-query softmax attention over every earlier key (the last m["window"] keys where the
    mixer names one); score(i, j) = q_i.k_j * scale * f(i) - r1 ln(1 + r2 (i - j)) (no bias without
    r1); the heads side by side times sigmoid(W_g h) where there is a W_g, then W_o."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[p + "q"].T).view(T, H, D)
    k = (h @ t[p + "k"].T).view(T, G, D)
    v = (h @ t[p + "v"].T).view(T, G, V)
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        g = head // (H // G)
        r1, r2 = (float(t[p + "r1"][head]), float(t[p + "r2"][head])) if p + "r1" in t else (0.0, 0.0)
        for i in range(T):
            qi = q[i, head] * query_factor(i, m.get("q_temp"))
            distance = torch.arange(i, -1, -1, dtype=F64)          # i - j for j = 0 .. i
            scores = (k[: i + 1, g] @ qi) * m["scale"] - r1 * torch.log(1.0 + r2 * distance)
            if m.get("window"):
                scores[distance >= m["window"]] = -math.inf
            w = torch.softmax(scores, 0)
            out[i, head] = w @ v[: i + 1, g]
    out = out.reshape(T, H * V)
    if p + "g" in t:
        out = out * torch.sigmoid(h @ t[p + "g"].T)
    return out @ t[p + "o"].T


# ------------------------------------------------------------------ the pair's right side
def gated_linear_recurrent_unit(h, m, t, p):
    """y = gelu(W_y h + b); u = conv(W_x h + b); r, i = sigmoid of a square matrix per part of u;
    log a = -8 r softplus(lam); S <- a S + sqrt(1 - a^2) i u from S = 0; W_o (S * y)."""
    T = h.shape[0]
    C, B = m["width"], m["blocks"]
    y = gelu_tanh(h @ t[p + "y"].T + t[p + "y.b"])
    u = causal_conv(h @ t[p + "x"].T + t[p + "x.b"], t[p + "conv"], t[p + "conv.b"])
    r = torch.zeros(T, C, dtype=F64)
    i = torch.zeros(T, C, dtype=F64)
    n = C // B
    for b in range(B):
        part = u[:, b * n:(b + 1) * n]
        r[:, b * n:(b + 1) * n] = torch.sigmoid(part @ t[p + "ra"][b].T + t[p + "ra.b"][b])
        i[:, b * n:(b + 1) * n] = torch.sigmoid(part @ t[p + "ri"][b].T + t[p + "ri.b"][b])
    a = torch.exp(-8.0 * r * softplus(t[p + "lam"]))
    S = torch.zeros(C, dtype=F64)
    states = torch.zeros(T, C, dtype=F64)
    for step in range(T):
        S = a[step] * S + torch.sqrt(1.0 - a[step] ** 2) * i[step] * u[step]
        states[step] = S
    return (states * y) @ t[p + "o"].T


def normed_pair(h, m, t, p, eps):
    left = distance_bias_attention(h, m["left"], t, p + "left.")
    right = gated_linear_recurrent_unit(h, m["right"], t, p + "right.")
    return 0.5 * (rms_norm(left, t[p + "left.out"], eps) + rms_norm(right, t[p + "right.out"], eps))


# ------------------------------------------------------------------ matrix states
def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def channel_delta_rule(h, m, t, p, eps):
    """Delta rule with a decay per value head and key channel; the read-out sees the token's own write."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ t[p + "q"].T, t[p + "q.conv"])).view(T, G, D)
    k = silu(causal_conv(h @ t[p + "k"].T, t[p + "k.conv"])).view(T, G, D)
    v = silu(causal_conv(h @ t[p + "v"].T, t[p + "v.conv"])).view(T, H, V)
    q, k = unit(q) * D ** -0.5, unit(k)
    beta = torch.sigmoid(h @ t[p + "b"].T)
    z = ((h @ t[p + "a1"].T) @ t[p + "a2"].T + t[p + "dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(t[p + "A_log"]).view(1, H, 1) * softplus(z))
    gate = torch.sigmoid((h @ t[p + "g1"].T) @ t[p + "g2"].T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(D, V, dtype=F64)
        for step in range(T):
            S = decay[step, head].unsqueeze(1) * S
            u = beta[step, head] * (v[step, head] - S.T @ k[step, g])
            S = S + torch.outer(k[step, g], u)
            o[step, head] = S.T @ q[step, g]
    o = rms_norm(o, t[p + "norm"], eps) * gate
    return o.reshape(T, H * V) @ t[p + "o"].T


def gated_linear_attention(h, m, t, p, eps):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (h @ t[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ t[p + "k"].T).view(T, H, D)
    v = (h @ t[p + "v"].T).view(T, H, V)
    z = (h @ t[p + "a1"].T) @ t[p + "a2"].T + t[p + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).view(T, H, D)
    o = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        S = torch.zeros(D, V, dtype=F64)
        for step in range(T):
            S = alpha[step, head].unsqueeze(1) * S + torch.outer(k[step, head], v[step, head])
            o[step, head] = S.T @ q[step, head]
    o = rms_norm(o, t[p + "norm"], eps).reshape(T, H * V) * silu(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


# ------------------------------------------------------------------ feed-forwards
def dense_mlp(h, t, p):
    return gelu_tanh(h @ t[p + "up"].T + t[p + "up.b"]) @ t[p + "down"].T + t[p + "down.b"]


def routed_experts(h, f, t, p):
    """softmax over all experts; the `top` largest, their scores as they are; squared relu inside."""
    scores = torch.softmax(h @ t[p + "router"].T, -1)
    out = torch.zeros_like(h)
    for row in range(h.shape[0]):
        order = sorted(range(f["router"]["experts"]), key=lambda e: (-float(scores[row, e]), e))
        for e in order[: f["router"]["top"]]:
            inner = torch.relu(h[row] @ t[p + f"e{e}.up"].T) ** 2
            out[row] += scores[row, e] * (inner @ t[p + f"e{e}.down"].T)
    return out


def feed_forward(h, f, t, p):
    if not f:
        return torch.zeros_like(h)
    return dense_mlp(h, t, p) if f["kind"] == "dense" else routed_experts(h, f, t, p)


# ------------------------------------------------------------------ what follows the sub-layers
def token_input(x, tokens, layer, dim, t, eps):
    p = f"l{layer}.side."
    e = t["side.embed"][torch.as_tensor(tokens, dtype=torch.long)][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ t[p + "gate"].T) * e) @ t[p + "proj"].T
    return x + rms_norm(y, t[p + "norm"], eps)


def depth_average(results, w):
    return sum(w[j] * results[j] for j in range(len(results)))


def mixer(h, spec, t, p, eps):
    if spec["type"] == "parallel":
        return normed_pair(h, spec["mixer"], t, p, eps)
    if spec["type"] == "channel_delta":
        return channel_delta_rule(h, spec["mixer"], t, p, eps)
    if spec["type"] == "gla":
        return gated_linear_attention(h, spec["mixer"], t, p, eps)
    raise ValueError(spec["type"])


def forward(config, tensors, tokens, return_layers=False):
    """Logits [T, vocab] (float64) of one request's tokens from position 0."""
    t = {k: v.to(F64) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)] * (config.get("embedding") or {}).get("scale", 1.0)
    results, after = [x], []
    for layer, spec in enumerate(config["layers"]):
        p = f"l{layer}."
        h = rms_norm(x, t[p + "norm1"], eps)
        x = x + (mixer(h, spec, t, p + "mix.", eps) + feed_forward(h, spec.get("mlp"), t, p + "mlp."))
        if config.get("token_side"):
            x = token_input(x, tokens, layer, config["token_side"]["dim"], t, eps)
        results.append(x)
        if p + "dwa" in t:
            x = depth_average(results, t[p + "dwa"])
        after.append(x.clone())
    logits = rms_norm(x, t["final.norm"], eps) @ t["head"].T
    return (logits, torch.stack(after)) if return_layers else logits


def greedy(config, tensors, prompt, n_new):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(config, tensors, tokens)[-1].argmax()))
    return tokens[len(prompt):]

"""Plain, slow float64 oracle of the Momedra design: one function per
mechanism, explicit loops over tokens and heads, no paging, no batching,
no state objects. It shares no code with fusioninfer_amd; tests compare
the engine (CPU ops or HIP kernels) against it.

Weights use the checkpoint naming (``l<i>.mix.q``, ``l<i>.mlp.e0.up`` ...),
as a dict of float64 tensors; ``cfg`` is the config.json dict.
"""

import math

import torch

F64 = torch.float64


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(
        math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def relu_sq(z):
    return torch.clamp(z, min=0.0) ** 2


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w, biased variance, no bias."""
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    var = (d * d).mean(-1, keepdim=True)
    return d / torch.sqrt(var + eps) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def rotate_pairs(x, pos, dims, base):
    """Interleaved pairs (2i, 2i+1) of the first ``dims`` entries of the
    vector x turned by pos * base^(-2i/dims); the rest pass."""
    y = x.clone()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        u, v = x[2 * i], x[2 * i + 1]
        y[2 * i] = u * math.cos(a) - v * math.sin(a)
        y[2 * i + 1] = v * math.cos(a) + u * math.sin(a)
    return y


def attend(q, K, V, scale, sink=None):
    """One query over the keys K [n, d] and values V [n, v]: softmax of
    (K q) * scale, with exp(sink) added to the denominator when given."""
    s = (K @ q) * scale
    mx = s.max() if sink is None else torch.maximum(s.max(), sink)
    e = torch.exp(s - mx)
    den = e.sum()
    if sink is not None:
        den = den + torch.exp(sink - mx)
    return ((e / den)[:, None] * V).sum(0)


def gated_attention(h, P, pre, m, eps):
    """Grouped-query softmax attention without rotation: biased
    projections, weighted RMS norm of every query and key head, a query
    factor growing with the logarithm of the position's block index, a
    sigmoid gate per head on the result."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], \
        m.get("vdim", m["dim"])
    q = (h @ P[pre + "q"].T + P[pre + "q.b"]).view(T, H, D)
    k = (h @ P[pre + "k"].T + P[pre + "k.b"]).view(T, G, D)
    v = (h @ P[pre + "v"].T + P[pre + "v.b"]).view(T, G, V)
    q = rms_norm(q, P[pre + "q.norm"], eps)
    k = rms_norm(k, P[pre + "k.norm"], eps)
    gate = sigmoid(h @ P[pre + "g"].T)                        # [T, H]
    qt = m.get("q_temp")
    out = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        temp = 1.0
        if qt:
            temp = 1.0 + qt["coef"] * math.log((t + 1) // qt["every"] + 1)
        for hh in range(H):
            g = hh // (H // G)
            s = (k[: t + 1, g] @ (q[t, hh] * temp)) * m["scale"]
            w = torch.softmax(s, 0)
            out[t, hh] = (w[:, None] * v[: t + 1, g]).sum(0) * gate[t, hh]
    return out.reshape(T, H * V) @ P[pre + "o"].T


def latent_attention(h, P, pre, m, eps):
    """Keys and values expanded from one normed low-rank latent per token;
    a rotated key part shared by all heads; softmax whose denominator
    holds one extra exp(sink) per head."""
    T = h.shape[0]
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], \
        m.get("vdim", m["dim"]), m["kv_rank"]
    base = m["rot"]["base"]
    dims = m["rot"].get("dims", R)      # leading entries of the part that turn
    q = (h @ P[pre + "q"].T).view(T, H, D + R)
    ckr = h @ P[pre + "dkv"].T
    c = rms_norm(ckr[:, :C], P[pre + "dkv.norm"], eps)
    kr = torch.stack([rotate_pairs(ckr[t, C:], t, dims, base)
                      for t in range(T)])
    ku = (c @ P[pre + "uk"].T).view(T, H, D)
    v = (c @ P[pre + "uv"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        for hh in range(H):
            qr = rotate_pairs(q[t, hh, D:], t, dims, base)
            s = (ku[: t + 1, hh] @ q[t, hh, :D] + kr[: t + 1] @ qr) \
                * m["scale"]
            e = torch.exp(s - s.max())
            den = e.sum() + torch.exp(P[pre + "sink"][hh] - s.max())
            out[t, hh] = ((e / den)[:, None] * v[: t + 1, hh]).sum(0)
    return out.reshape(T, H * V) @ P[pre + "o"].T


def causal_conv(x, w, b):
    """y[t, c] = b[c] + sum_j w[c, j] x[t - (taps-1) + j, c], zeros before
    the start."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        y[t] = b
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


def rglru_mixer(h, P, pre, m):
    """Gated linear recurrence per channel: a gelu branch times the state
    of S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t, a_t = exp(-8 r_t
    softplus(lam)), with r and i from block-diagonal sigmoid gates of the
    convolved branch u."""
    T = h.shape[0]
    W, B = m["width"], m["blocks"]
    y = gelu_tanh(h @ P[pre + "y"].T + P[pre + "y.b"])
    u = causal_conv(h @ P[pre + "x"].T + P[pre + "x.b"], P[pre + "conv"],
                    P[pre + "conv.b"])
    bw = W // B
    r = torch.zeros(T, W, dtype=F64)
    i = torch.zeros(T, W, dtype=F64)
    for b in range(B):
        ub = u[:, b * bw: (b + 1) * bw]
        r[:, b * bw: (b + 1) * bw] = sigmoid(
            ub @ P[pre + "ra"][b].T + P[pre + "ra.b"][b])
        i[:, b * bw: (b + 1) * bw] = sigmoid(
            ub @ P[pre + "ri"][b].T + P[pre + "ri.b"][b])
    S = torch.zeros(W, dtype=F64)
    out = torch.zeros(T, W, dtype=F64)
    sp = softplus(P[pre + "lam"])
    for t in range(T):
        a = torch.exp(-8.0 * r[t] * sp)
        S = a * S + torch.sqrt(1.0 - a * a) * i[t] * u[t]
        out[t] = S * y[t]
    return out @ P[pre + "o"].T


def dense_ff(h, P, pre):
    return relu_sq(h @ P[pre + "up"].T) @ P[pre + "down"].T


def moe_ff(h, P, pre, m):
    """Top experts by router logit, weights = softmax over the chosen
    logits only; a shared expert added for every token."""
    T = h.shape[0]
    E, top = m["router"]["experts"], m["router"]["top"]
    z = h @ P[pre + "router"].T + P[pre + "router.b"]
    out = torch.zeros(T, P[pre + "e0.down"].shape[0], dtype=F64)
    for t in range(T):
        idx = torch.argsort(z[t], descending=True)[:top]
        w = torch.softmax(z[t, idx], 0)
        for j, e in enumerate(idx.tolist()):
            out[t] += w[j] * dense_ff(h[t], P, f"{pre}e{e}.")
    if m.get("shared"):
        out = out + dense_ff(h, P, pre + "shared.")
    return out


def feed_forward(h, P, pre, m):
    if m is None:
        return torch.zeros_like(h)
    if m["kind"] == "dense":
        return dense_ff(h, P, pre)
    return moe_ff(h, P, pre, m)


def mixer(kind, h, P, pre, m, eps):
    if kind == "attention":
        return gated_attention(h, P, pre, m, eps)
    if kind == "latent_attention":
        return latent_attention(h, P, pre, m, eps)
    if kind == "rglru":
        return rglru_mixer(h, P, pre, m)
    raise ValueError(kind)


def layer_runs(cfg):
    """Layer indices in execution order, with a marker where a pass of the
    repeated span begins."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    runs += [(i, False) for i in range(b, n)]
    return runs


def forward(tokens, P, cfg, return_layers=False):
    eps = cfg["norm"]["eps"]
    mult = cfg.get("residual_mult", 1.0)
    x0 = P["embed"][torch.as_tensor(tokens)]
    x = x0.clone()
    layers = []
    for i, enters in layer_runs(cfg):
        L = cfg["layers"][i]
        if enters:
            x = torch.cat([x, x0], -1) @ P["loop.in"].T
        h = layer_norm(x, P[f"l{i}.norm1"], eps)
        x = x + mult * (mixer(L["type"], h, P, f"l{i}.mix.", L["mixer"], eps)
                        + feed_forward(h, P, f"l{i}.mlp.", L.get("mlp")))
        layers.append(x.clone())
    logits = layer_norm(x, P["final.norm"], eps) @ P["head"].T
    if return_layers:
        return logits, torch.stack(layers)
    return logits


def greedy(tokens, P, cfg, n_new):
    toks = list(tokens)
    for _ in range(n_new):
        toks.append(int(forward(toks, P, cfg)[-1].argmax()))
    return toks[len(tokens):]

"""Plain, slow float64 oracle of the Kazozen design: one function per
mechanism, explicit loops over tokens and heads, no paging, no batching,
no state objects. It shares no code with fusioninfer_amd; tests compare
the engine (CPU ops or HIP kernels) against it.

Weights use the checkpoint naming (``l<i>.mix.q`` ...), as a dict of
float64 tensors; ``cfg`` is the config.json dict.

The design in short: token embedding times a constant plus a hashed
(previous token, token) table row; layers ``x += LN(mixer(x))``,
``x += LN(ff(x))`` (the norm sits on the sublayer's OUTPUT); the mixer is
grouped-query attention with projection biases, an RMS norm over the whole
q / k projection, interleaved partial rotary positions with a YaRN
frequency blend, a sliding window that always keeps the first tokens, a
per-head sink in the softmax denominator and an elementwise sigmoid gate;
a layer may borrow the keys and values of an earlier layer; the
feed-forward is a clamped gated unit, dense or as group-limited routed
experts; the tied head's logits go through a tanh cap.
"""

import math

import torch

F64 = torch.float64


def layer_norm_wb(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def bigram_row(prev, tok, bg):
    """Row of the pair table for (prev, tok); prev None at a sequence's
    first token: the extra last row."""
    if prev is None:
        return bg["buckets"]
    return (prev * bg["mul_prev"] + tok * bg["mul_cur"]) % bg["buckets"]


def embed_tokens(tokens, W, cfg, prev=None):
    e = cfg.get("embedding") or {}
    rows = []
    for t in tokens:
        x = W["embed"][t] * float(e.get("scale", 1.0))
        if e.get("bigram"):
            x = x + W["bigram"][bigram_row(prev, t, e["bigram"])]
        rows.append(x)
        prev = t
    return torch.stack(rows)


def rotary_frequencies(rot):
    """([dims/2] angular frequencies, factor on cos and sin)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor = float(sc["factor"])

    def turn_index(turns):
        return (dims * math.log(sc["original"] / (2.0 * math.pi * turns))
                / (2.0 * math.log(base)))

    lo = max(math.floor(turn_index(sc["fast"])), 0)
    hi = min(math.ceil(turn_index(sc["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x, pos, freqs, mult):
    """x: [heads, D]; pairs (2i, 2i+1) for i < len(freqs) turn by
    pos * freqs[i]; cos and sin carry the factor ``mult``."""
    y = x.clone()
    for i, f in enumerate(freqs):
        c, s = math.cos(pos * f) * mult, math.sin(pos * f) * mult
        a, b = x[:, 2 * i], x[:, 2 * i + 1]
        y[:, 2 * i] = a * c - b * s
        y[:, 2 * i + 1] = b * c + a * s
    return y


def sees(i, j, mask):
    if j > i:
        return False
    if not mask or not mask.get("size"):
        return True
    return i - j < mask["size"] or j < mask.get("keep_first", 0)


def keys_values(h, W, pre, m, eps, pos0=0):
    """Cached form of the keys (normed, rotated) [T, G, dim] and the values
    [T, G, vdim] of rows h at positions pos0.."""
    G, D, V = m["kv_heads"], m["dim"], m["vdim"]
    k = h @ W[pre + "k"].T + W[pre + "k.b"]
    v = h @ W[pre + "v"].T + W[pre + "v.b"]
    k = unit_rms(k, eps) * W[pre + "k.norm"]
    freqs, mult = rotary_frequencies(m["rot"]) if m.get("rot") else ([], 1.0)
    ks = torch.stack([rotate_interleaved(k[t].reshape(G, D), pos0 + t,
                                         freqs, mult)
                      for t in range(h.shape[0])])
    return ks, v.reshape(-1, G, V)


def attend_row(q, ks, vs, p, mask, scale, sinks):
    """One query row q [H, D] at position p over keys ks [>=p+1, G, D] and
    values vs [>=p+1, G, V]; returns [H, V]."""
    H, G = q.shape[0], ks.shape[1]
    js = [j for j in range(p + 1) if sees(p, j, mask)]
    out = []
    for hh in range(H):
        g = hh // (H // G)
        sc = (ks[js, g] @ q[hh]) * scale
        top = torch.maximum(sc.max(), sinks[hh])
        ex = torch.exp(sc - top)
        den = ex.sum() + torch.exp(sinks[hh] - top)
        out.append((ex / den) @ vs[js, g])
    return torch.stack(out)


def queries(h, W, pre, m, eps, pos0=0):
    """Normed, rotated queries [T, H, dim] of rows h at positions pos0.."""
    H, D = m["heads"], m["dim"]
    q = h @ W[pre + "q"].T + W[pre + "q.b"]
    q = unit_rms(q, eps) * W[pre + "q.norm"]
    freqs, mult = rotary_frequencies(m["rot"]) if m.get("rot") else ([], 1.0)
    return torch.stack([rotate_interleaved(q[t].reshape(H, D), pos0 + t,
                                           freqs, mult)
                        for t in range(h.shape[0])])


def attention_mixer(h, W, pre, m, eps, kv, pos0=0):
    """h: rows at positions pos0..; kv = (keys, values) of positions 0..
    (the layer's own or the borrowed ones). Returns the projected output."""
    T = h.shape[0]
    q = queries(h, W, pre, m, eps, pos0)
    gate = torch.sigmoid(h @ W[pre + "g"].T)
    ks, vs = kv
    out = torch.stack([
        attend_row(q[t], ks, vs, pos0 + t, m.get("mask"), m["scale"],
                   W[pre + "sink"]).reshape(-1) for t in range(T)])
    return (out * gate) @ W[pre + "o"].T


def clamped_glu(g, u, limit):
    g = torch.clamp(g, max=limit)
    u = torch.clamp(u, -limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def gated_unit(h, W, pre, limit):
    y = clamped_glu(h @ W[pre + "gate"].T, h @ W[pre + "up"].T, limit)
    return y @ W[pre + "down"].T


def route(z, correction, r):
    """z: router logits of ONE token. Returns [(expert, weight)]."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(z)
    c = s + correction
    allowed = list(range(E))
    gr = r.get("groups")
    if gr:
        n = E // gr["count"]
        score = []
        for a in range(gr["count"]):
            best = sorted((float(c[e]) for e in range(a * n, (a + 1) * n)),
                          reverse=True)[:2]
            score.append(sum(best))
        keep = sorted(range(gr["count"]), key=lambda a: (-score[a], a))
        keep = keep[: gr["keep"]]
        allowed = [e for e in range(E) if e // n in keep]
    chosen = sorted(allowed, key=lambda e: (-float(c[e]), e))[:top]
    return [(e, s[e]) for e in chosen]


def routed_experts(h, W, pre, mlp):
    out = torch.zeros(h.shape[0], W[pre + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        z = W[pre + "router"] @ h[t]
        for e, w in route(z, W[pre + "correction"], mlp["router"]):
            out[t] += w * gated_unit(h[t:t + 1], W, f"{pre}e{e}.",
                                     mlp["expert"]["limit"])[0]
    return out


def feed_forward(h, W, pre, mlp):
    if mlp["kind"] == "dense":
        return gated_unit(h, W, pre, mlp["limit"])
    return routed_experts(h, W, pre, mlp)


def forward(tokens, W, cfg, trace=None):
    """Whole sequence from position 0; returns capped logits [T, vocab].
    ``trace``: list that receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = embed_tokens(tokens, W, cfg)
    held = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = L["mixer"]
        src = m.get("kv_from")
        if src is None:
            held[i] = keys_values(x, W, p + "mix.", m, eps)
            src = i
        y = attention_mixer(x, W, p + "mix.", m, eps, held[src])
        x = x + layer_norm_wb(y, W[p + "norm1"], W[p + "norm1.b"], eps)
        if L.get("mlp"):
            y = feed_forward(x, W, p + "mlp.", L["mlp"])
            x = x + layer_norm_wb(y, W[p + "norm2"], W[p + "norm2.b"], eps)
        if trace is not None:
            trace.append(x.clone())
    h = layer_norm_wb(x, W["final.norm"], W["final.norm.b"], eps)
    logits = h @ W["embed"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits


def greedy(prompt, W, cfg, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(forward(toks, W, cfg)[-1].argmax()))
    return toks[len(prompt):]

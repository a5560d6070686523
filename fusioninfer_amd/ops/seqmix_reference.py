"""PyTorch implementations of the sequence-mixer ops (ops/seqmix.py).

These are the CPU execution path and the numerics oracle the HIP kernels
of ``_C_seqmix`` are tested against. Everything that the kernels keep in
32-bit (norm statistics, residual stream, rotary angles, attention scores
and softmax, decays, gates and the recurrent state) is fp32 here as well;
``out_dtype`` only rounds what is handed to the next matrix product.

Batch layout shared by all ops: the step's token rows are grouped by
sequence, ``seq_cu[s]:seq_cu[s+1]`` are the rows of sequence ``s`` (a
decoding sequence is a one-row group), ``row_seq[t]`` is the group of row
``t``, ``positions[t]`` its absolute position, ``seq_slots[s]`` the
sequence's state slot (-1: no state kept) and ``seq_bt[s]`` its block
table into the paged cache.
"""

from __future__ import annotations

import math

import torch


def _rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def scalar_rms_norm(x, g, eps: float, out_dtype):
    """x / sqrt(mean(x^2) + eps) * g with ONE gain for all coordinates."""
    return (_rms(x.float(), eps) * g.float()).to(out_dtype)


def residual_add_scalar_norm_(resid, y, g_post, eps: float, g_next=None,
                              out_dtype=None):
    """resid += rms(y) * g_post (fp32, in place); optionally returns the
    next sublayer's input rms(resid) * g_next."""
    resid.add_(_rms(y.float(), eps) * g_post.float())
    if g_next is None:
        return None
    return (_rms(resid, eps) * g_next.float()).to(out_dtype)


def norm_token_shift(resid, g, shift, state, seq_cu, row_seq, positions,
                     seq_slots, eps: float, out_dtype):
    """h = rms(resid) * g, then every row is pulled towards the previous
    token's h: h + (h_prev - h) * shift. The previous token of a group's
    first row comes from ``state`` (zeros at position 0); the group's last
    h is stored back."""
    h = _rms(resid, eps) * g.float()
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    cu = seq_cu.tolist()
    slots = seq_slots.tolist()
    pos = positions.tolist()
    for s in range(len(slots)):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        if pos[a] == 0 or slots[s] < 0:
            prev[a] = 0
        else:
            prev[a] = state[slots[s]]
        if slots[s] >= 0:
            state[slots[s]] = h[b - 1]
    return (h + (prev - h) * shift.float()).to(out_dtype)


def rope_unitnorm_cache_(q, k, positions, inv_freq, eps: float, k_cache,
                         v_cache, slot_mapping, num_heads: int,
                         num_kv_heads: int, head_dim: int):
    """Interleaved-pair rotary embedding on the first 2*len(inv_freq)
    dims of every q/k head, then each head divided by its RMS (no gain).
    The UNPROCESSED k rows go to ``v_cache`` (shared key/value projection),
    the processed ones to ``k_cache``. Returns processed q [T, H, D]."""
    T = q.shape[0]
    qf = q.float().reshape(T, num_heads, head_dim)
    kf = k.float().reshape(T, num_kv_heads, head_dim)
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    rd = 2 * inv_freq.numel()

    def rot(t):
        t = t.clone()
        u, w = t[..., 0:rd:2].clone(), t[..., 1:rd:2].clone()
        t[..., 0:rd:2] = u * c - w * s
        t[..., 1:rd:2] = w * c + u * s
        return t

    qo = _rms(rot(qf), eps)
    ko = _rms(rot(kf), eps)
    bs = k_cache.shape[2]
    slots = slot_mapping.long()
    ok = slots >= 0
    blk, off = slots[ok] // bs, slots[ok] % bs
    k_cache[blk, :, off, :] = ko[ok].to(k_cache.dtype)
    v_cache[blk, :, off, :] = kf[ok].to(v_cache.dtype)
    return qo.to(q.dtype)


def ranged_paged_attention(q, k_cache, v_cache, seq_bt, row_seq, positions,
                           scale: float, chunk: int = 0, window: int = 0):
    """Softmax attention of every row over the paged keys of its own
    sequence at positions lo..p, where p is the row's position and lo is
    the start of p's chunk (``chunk`` > 0: chunks of that many positions
    counted from 0) and/or p - window + 1 (``window`` > 0)."""
    T, H, D = q.shape
    G, bs = k_cache.shape[1], k_cache.shape[2]
    rep = H // G
    out = torch.zeros(T, H, v_cache.shape[3], dtype=torch.float32)
    pos = positions.tolist()
    rs = row_seq.tolist()
    qf = q.float()
    t = 0
    while t < T:
        # rows of one sequence that share a key range start are batched
        s = rs[t]
        e = t
        while e + 1 < T and rs[e + 1] == s:
            e += 1
        p0, p1 = pos[t], pos[e]
        lo_all = 0
        if chunk > 0:
            lo_all = (p0 // chunk) * chunk
        if window > 0:
            lo_all = max(lo_all, p0 - window + 1)
        idx = torch.arange(lo_all, p1 + 1)
        blocks = seq_bt[s].long()[idx // bs]
        kk = k_cache[blocks, :, idx % bs, :].float()   # [L, G, D]
        vv = v_cache[blocks, :, idx % bs, :].float()
        kk = kk.repeat_interleave(rep, dim=1)
        vv = vv.repeat_interleave(rep, dim=1)
        pr = torch.tensor(pos[t:e + 1])
        sc = torch.einsum("ihd,jhd->hij", qf[t:e + 1], kk) * scale
        vis = idx[None, :] <= pr[:, None]
        if chunk > 0:
            vis &= (idx[None, :] // chunk) == (pr[:, None] // chunk)
        if window > 0:
            vis &= idx[None, :] > (pr[:, None] - window)
        sc = sc.masked_fill(~vis[None], float("-inf"))
        w = torch.softmax(sc, dim=-1)
        out[t:e + 1] = torch.einsum("hij,jhd->ihd", w, vv)
        t = e + 1
    return out.to(q.dtype)


def delta_rule(r, k, v, wlin, alin, glin, w0, a_bias, norm_w, state,
               seq_cu, seq_slots, positions, heads: int, dim: int,
               eps: float, decay_scale: float):
    """Generalized delta rule with per-channel decay and removal rate.

    Per head, with u = k / sqrt(|k|^2 + 1e-6),
    w = exp(-decay_scale * sigmoid(wlin + w0)), a = sigmoid(alin + a_bias):
        S <- diag(w) S - (a*u) (u^T S) + k v^T      (both terms read old S)
        o  = S^T r
    o is divided by its RMS per head, scaled by norm_w and sigmoid(glin).
    ``state`` [slots, heads, dim, dim] fp32 carries S between steps (zero
    at position 0)."""
    T = r.shape[0]
    rf = r.float().reshape(T, heads, dim)
    kf = k.float().reshape(T, heads, dim)
    vf = v.float().reshape(T, heads, dim)
    w = torch.exp(-decay_scale * torch.sigmoid(wlin.float() + w0.float()))
    w = w.reshape(T, heads, dim)
    a = torch.sigmoid(alin.float() + a_bias.float()).reshape(T, heads, dim)
    u = kf * torch.rsqrt(kf.pow(2).sum(dim=-1, keepdim=True) + 1e-6)
    au = a * u
    o = torch.empty(T, heads, dim, dtype=torch.float32)
    cu = seq_cu.tolist()
    slots = seq_slots.tolist()
    pos = positions.tolist()
    for s in range(len(slots)):
        a0, b0 = cu[s], cu[s + 1]
        if b0 <= a0:
            continue
        if pos[a0] == 0 or slots[s] < 0:
            S = torch.zeros(heads, dim, dim, dtype=torch.float32)
        else:
            S = state[slots[s]].clone()
        for t in range(a0, b0):
            uS = torch.einsum("hi,hij->hj", u[t], S)
            S = (w[t][:, :, None] * S - au[t][:, :, None] * uS[:, None, :]
                 + kf[t][:, :, None] * vf[t][:, None, :])
            o[t] = torch.einsum("hij,hi->hj", S, rf[t])
        if slots[s] >= 0:
            state[slots[s]] = S
    o = _rms(o, eps).reshape(T, heads * dim)
    o = o * norm_w.float() * torch.sigmoid(glin.float())
    return o.to(r.dtype)


def dual_norm_combine_residual_(resid, yl, yr, wl, wr, g_post, eps: float,
                                g_next=None, out_dtype=None):
    """y = (rms(yl) * wl + rms(yr) * wr) / 2; resid += rms(y) * g_post;
    optionally returns rms(resid) * g_next."""
    y = 0.5 * (_rms(yl.float(), eps) * wl.float()
               + _rms(yr.float(), eps) * wr.float())
    resid.add_(_rms(y, eps) * g_post.float())
    if g_next is None:
        return None
    return (_rms(resid, eps) * g_next.float()).to(out_dtype)


def gelu_tanh_and_mul(gu):
    """gu: [T, 2F] (gate | up) -> gelu_tanh(gate) * up."""
    g, u = gu.float().chunk(2, dim=-1)
    act = 0.5 * g * (1.0 + torch.tanh(
        math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g)))
    return (act * u).to(gu.dtype)


# ------------------------------------------------------------------------
# Layer-norm residual stream with sigmoid-gated sublayer results, linear
# attention with a scalar decay per head, windowed softmax attention with
# a log-distance penalty and head mixing, the gated delta rule behind a
# short causal convolution, grouped unit-RMS output gates.

def layer_norm(x, w, eps: float, out_dtype):
    """(x - mean) / sqrt(var + eps) * w over the last dim (biased
    variance, no bias)."""
    xf = x.float()
    d = xf - xf.mean(dim=-1, keepdim=True)
    var = d.pow(2).mean(dim=-1, keepdim=True)
    return (d * torch.rsqrt(var + eps) * w.float()).to(out_dtype)


def gated_residual_layer_norm_(resid, y1, s1: float, y2, s2: float, gate_lin,
                               gate_bias, w_next, eps: float, out_dtype):
    """resid += (s1*y1 [+ s2*y2]) * sigmoid(gate_lin + gate_bias) in fp32,
    in place; optionally returns layer_norm(resid) * w_next."""
    y = y1.float() * s1
    if y2 is not None:
        y = y + y2.float() * s2
    resid.add_(y * torch.sigmoid(gate_lin.float() + gate_bias.float()))
    if w_next is None:
        return None
    return layer_norm(resid, w_next, eps, out_dtype)


def _group_state(state, slot, pos0, shape):
    if slot < 0 or pos0 == 0:
        return torch.zeros(shape, dtype=torch.float32)
    return state[slot].clone()


def decay_linear_attention(q, k, v, decay, state, seq_cu, seq_slots,
                           positions, heads: int, dim: int, vdim: int,
                           silu: bool = True):
    """Per head S_t = decay_h * S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with
    q/k/v passed through silu first when ``silu``. ``state``
    [slots, heads, dim, vdim] fp32 carries S between steps (zero at
    position 0). Returns the raw fp32 read-outs [T, heads*vdim]."""
    T = q.shape[0]
    act = torch.nn.functional.silu if silu else (lambda z: z)
    qf = act(q.float()).reshape(T, heads, dim)
    kf = act(k.float()).reshape(T, heads, dim)
    vf = act(v.float()).reshape(T, heads, vdim)
    lam = decay.float().reshape(heads, 1, 1)
    o = torch.empty(T, heads, vdim, dtype=torch.float32)
    cu, slots, pos = seq_cu.tolist(), seq_slots.tolist(), positions.tolist()
    for s in range(len(slots)):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        S = _group_state(state, slots[s], pos[a], (heads, dim, vdim))
        for t in range(a, b):
            S = lam * S + kf[t][:, :, None] * vf[t][:, None, :]
            o[t] = torch.einsum("hij,hi->hj", S, qf[t])
        if slots[s] >= 0:
            state[slots[s]] = S
    return o.reshape(T, heads * vdim)


def group_rms_gate(o_raw, glin, w, groups: int, eps: float, gate: str,
                   out_dtype):
    """Rows of o_raw [T, N] are cut into ``groups`` equal parts, each
    divided by its root mean square; then times ``w`` ([N], or one part's
    worth shared by all parts) and sigmoid or silu of glin."""
    T, N = o_raw.shape
    part = N // groups
    o = _rms(o_raw.float().reshape(T, groups, part), eps)
    wf = w.float()
    o = o * (wf.reshape(1, 1, part) if wf.numel() == part
             else wf.reshape(1, groups, part))
    g = glin.float().reshape(T, groups, part)
    g = torch.sigmoid(g) if gate == "sigmoid" else \
        torch.nn.functional.silu(g)
    return (o * g).reshape(T, N).to(out_dtype)


def paged_cache_write_(k, v, k_cache, v_cache, slot_mapping):
    """Rows of k [T, G*D] / v [T, G*V] into k_cache [B, G, bs, D] /
    v_cache [B, G, bs, V] at slot_mapping (negative: skipped)."""
    T = k.shape[0]
    G, bs = k_cache.shape[1], k_cache.shape[2]
    slots = slot_mapping.long()
    ok = slots >= 0
    blk, off = slots[ok] // bs, slots[ok] % bs
    k_cache[blk, :, off, :] = k.reshape(T, G, -1)[ok].to(k_cache.dtype)
    v_cache[blk, :, off, :] = v.reshape(T, G, -1)[ok].to(v_cache.dtype)


def talking_window_attention(q, k_cache, v_cache, seq_bt, row_seq, positions,
                             scale: float, window: int, r1, r2, talk):
    """Softmax attention over the paged keys j of the row's own sequence
    with 0 <= p - j < window (window <= 0: all j <= p). Per head the raw
    score is (q.k)*scale - r1_h * ln(1 + r2_h * (p - j)); the heads'
    scores are then mixed, score_h <- sum_g talk[h, g] score_g, before
    the softmax. q: [T, H, D]; returns [T, H, V]."""
    T, H, D = q.shape
    G, bs = k_cache.shape[1], k_cache.shape[2]
    rep = H // G
    out = torch.zeros(T, H, v_cache.shape[3], dtype=torch.float32)
    pos = positions.tolist()
    rs = row_seq.tolist()
    qf = q.float()
    r1f, r2f, tk = r1.float(), r2.float(), talk.float()
    t = 0
    while t < T:
        s = rs[t]
        e = t
        while e + 1 < T and rs[e + 1] == s:
            e += 1
        p0, p1 = pos[t], pos[e]
        lo = max(p0 - window + 1, 0) if window > 0 else 0
        idx = torch.arange(lo, p1 + 1)
        blocks = seq_bt[s].long()[idx // bs]
        kk = k_cache[blocks, :, idx % bs, :].float()
        vv = v_cache[blocks, :, idx % bs, :].float()
        kk = kk.repeat_interleave(rep, dim=1)
        vv = vv.repeat_interleave(rep, dim=1)
        pr = torch.tensor(pos[t:e + 1])
        dist = (pr[:, None] - idx[None, :])                  # [rows, keys]
        vis = dist >= 0
        if window > 0:
            vis &= dist < window
        sc = torch.einsum("ihd,jhd->hij", qf[t:e + 1], kk) * scale
        dpos = dist.clamp(min=0).float()
        sc = sc - r1f[:, None, None] * torch.log1p(
            r2f[:, None, None] * dpos[None])
        sc = torch.einsum("hg,gij->hij", tk, sc)
        sc = sc.masked_fill(~vis[None], float("-inf"))
        w = torch.softmax(sc, dim=-1)
        out[t:e + 1] = torch.einsum("hij,jhd->ihd", w, vv)
        t = e + 1
    return out.to(q.dtype)


def gated_delta_rule(x, conv_w, alin, blin, a_log, dt_bias, conv_state,
                     state, seq_cu, seq_slots, positions, heads: int,
                     kv_heads: int, dim: int, vdim: int):
    """Gated delta rule behind a short causal convolution.

    x [T, C] holds the projections q | k | v (kv_heads*dim, kv_heads*dim,
    heads*vdim channels). Every channel passes a causal convolution over
    time (conv_w [C, taps], last column = current token, zeros before the
    sequence start) and silu; q and k become unit vectors per head
    (x / sqrt(|x|^2 + 1e-6)), q times dim^-0.5. With beta = sigmoid(blin)
    and g = exp(-exp(a_log) * softplus(alin + dt_bias)), per head

        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.

    Head h reads q/k head h // (heads // kv_heads). ``conv_state``
    [slots, taps-1, C] fp32 keeps the last taps-1 inputs, ``state``
    [slots, heads, dim, vdim] fp32 keeps S. Returns raw fp32 o
    [T, heads*vdim]."""
    T, C = x.shape
    taps = conv_w.shape[1]
    nq = kv_heads * dim
    xf = x.float()
    wf = conv_w.float()
    rep = heads // kv_heads
    beta = torch.sigmoid(blin.float())
    g = torch.exp(-torch.exp(a_log.float())
                  * torch.nn.functional.softplus(alin.float()
                                                 + dt_bias.float()))
    o = torch.empty(T, heads, vdim, dtype=torch.float32)
    cu, slots, pos = seq_cu.tolist(), seq_slots.tolist(), positions.tolist()
    for s in range(len(slots)):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        slot, p0 = slots[s], pos[a]
        hist = torch.zeros(taps - 1, C, dtype=torch.float32)
        if slot >= 0 and p0 > 0 and taps > 1:
            hist = conv_state[slot].clone()
            # entries older than the sequence start count as zeros
            if p0 < taps - 1:
                hist[: taps - 1 - p0] = 0
        ext = torch.cat([hist, xf[a:b]], dim=0)              # [taps-1+n, C]
        y = torch.zeros(b - a, C, dtype=torch.float32)
        for j in range(taps):
            y += wf[:, j] * ext[j: j + (b - a)]
        y = torch.nn.functional.silu(y)
        if slot >= 0 and taps > 1:
            conv_state[slot] = ext[-(taps - 1):]
        qh = y[:, :nq].reshape(-1, kv_heads, dim)
        kh = y[:, nq:2 * nq].reshape(-1, kv_heads, dim)
        vh = y[:, 2 * nq:].reshape(-1, heads, vdim)
        qh = qh * torch.rsqrt(qh.pow(2).sum(-1, keepdim=True) + 1e-6) \
            * dim ** -0.5
        kh = kh * torch.rsqrt(kh.pow(2).sum(-1, keepdim=True) + 1e-6)
        qh = qh.repeat_interleave(rep, dim=1)
        kh = kh.repeat_interleave(rep, dim=1)
        S = _group_state(state, slot, p0, (heads, dim, vdim))
        for i in range(b - a):
            t = a + i
            S = g[t][:, None, None] * S
            u = beta[t][:, None] * (vh[i] - torch.einsum(
                "hij,hi->hj", S, kh[i]))
            S = S + kh[i][:, :, None] * u[:, None, :]
            o[t] = torch.einsum("hij,hi->hj", S, qh[i])
        if slot >= 0:
            state[slot] = S
    return o.reshape(T, heads * vdim)


# ------------------------------------------------------------------------
# parallel-residual stream, weighted head norms with a query temperature,
# latent (low-rank) keys/values with a shared rotated part and a softmax
# sink, gated linear recurrence behind a short convolution, squared relu.

def scaled_residual_layer_norm_(resid, ys, scales, w_next, eps: float,
                                out_dtype):
    """resid += sum_i scales[i] * ys[i] in fp32, in place; optionally
    returns layer_norm(resid) * w_next."""
    acc = None
    for y, s in zip(ys, scales):
        term = y.float() * s
        acc = term if acc is None else acc + term
    resid.add_(acc)
    if w_next is None:
        return None
    return layer_norm(resid, w_next, eps, out_dtype)


def cast_layer_norm(y, w_next, eps: float):
    """The fp32 stream restarted from an activation: returns (y as fp32
    copy, layer_norm(y) * w_next in y's dtype, or None without w_next)."""
    resid = y.to(torch.float32, copy=True)
    if w_next is None:
        return resid, None
    return resid, layer_norm(resid, w_next, eps, y.dtype)


def concat_cast(resid, x0):
    """[resid rounded to x0's dtype | x0] along the last dim."""
    return torch.cat([resid.to(x0.dtype), x0], dim=-1)


def query_temperature(positions, coef: float, every: int):
    """1 + coef * ln(floor((p + 1) / every) + 1) per row, fp32 (1 when
    every <= 0)."""
    if every <= 0 or coef == 0.0:
        return torch.ones(positions.shape[0], dtype=torch.float32)
    blk = torch.div(positions.long() + 1, every, rounding_mode="floor")
    return 1.0 + coef * torch.log((blk + 1).float())


def headnorm_qtemp_cache_(q, k, v, positions, q_w, k_w, eps: float,
                          temp_coef: float, temp_every: int, k_cache,
                          v_cache, slot_mapping, num_heads: int,
                          num_kv_heads: int, dim: int, vdim: int):
    """Every query and key head is divided by its root mean square and
    multiplied by a weight vector shared by all heads (q_w / k_w, [dim]);
    queries are then multiplied by the position's temperature. Normed keys
    and the unchanged values go to the paged caches; returns the
    processed queries [T, H, dim]."""
    T = q.shape[0]
    qf = _rms(q.float().reshape(T, num_heads, dim), eps) * q_w.float()
    kf = _rms(k.float().reshape(T, num_kv_heads, dim), eps) * k_w.float()
    qf = qf * query_temperature(positions, temp_coef,
                                temp_every).reshape(T, 1, 1)
    paged_cache_write_(kf.reshape(T, -1).to(q.dtype), v, k_cache, v_cache,
                       slot_mapping)
    return qf.to(q.dtype)


def _rotate_interleaved(x, ang):
    """Pairs (2i, 2i+1) of the last dim of x turned by ang[..., i]; pairs
    beyond the angles given pass unchanged."""
    n = 2 * ang.shape[-1]
    cs, sn = torch.cos(ang), torch.sin(ang)
    u, w = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = u * cs - w * sn
    out[..., 1:n:2] = w * cs + u * sn
    return out


def latent_rope_cache_(q, ckr, positions, inv_freq, norm_w, eps: float,
                       kv_cache, slot_mapping, num_heads: int, dim: int,
                       rot_dim: int, rank: int, q_out):
    """q [T, H*(dim+rot_dim)]: the trailing rot_dim entries of every head
    are rotated (interleaved pairs, fp32 angle = position * inv_freq; pairs
    beyond len(inv_freq) pass) and
    written to q_out[:, :, rank:]. ckr [T, rank+rot_dim]: the leading rank
    entries are RMS-normed with norm_w, the trailing rot_dim rotated; the
    row goes to kv_cache [B, 1, bs, rank+rot_dim] at slot_mapping."""
    T = q.shape[0]
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    qr = q.float().reshape(T, num_heads, dim + rot_dim)[:, :, dim:]
    q_out[:, :, rank:] = _rotate_interleaved(qr, ang[:, None, :]).to(
        q_out.dtype)
    cf = ckr.float()
    row = torch.cat([_rms(cf[:, :rank], eps) * norm_w.float(),
                     _rotate_interleaved(cf[:, rank:], ang)], dim=-1)
    bs = kv_cache.shape[2]
    slots = slot_mapping.long()
    ok = slots >= 0
    kv_cache[slots[ok] // bs, 0, slots[ok] % bs, :] = row[ok].to(
        kv_cache.dtype)


def sink_paged_attention(q, k_cache, v_cache, seq_bt, row_seq, positions,
                         scale: float, sink=None, value_dims: int = 0,
                         out_gate=None, window: int = 0, keep_first: int = 0):
    """Causal softmax attention of every row over the paged keys 0..p of
    its own sequence. ``sink`` [H] fp32: exp(sink_h) joins the softmax
    denominator (no key, no value). ``v_cache`` None: the values are the
    leading ``value_dims`` entries of the cached keys. ``out_gate`` [T, H]
    or [T, H*Dv]: head results (or every entry) are multiplied by
    sigmoid(out_gate). ``window`` > 0: key j is visible from position p
    only if p - j < window or j < keep_first. q [T, H, Dk]; returns
    [T, H, Dv]."""
    T, H, D = q.shape
    G, bs = k_cache.shape[1], k_cache.shape[2]
    rep = H // G
    V = v_cache.shape[3] if v_cache is not None else int(value_dims)
    out = torch.zeros(T, H, V, dtype=torch.float32)
    pos = positions.tolist()
    rs = row_seq.tolist()
    qf = q.float()
    t = 0
    while t < T:
        s = rs[t]
        e = t
        while e + 1 < T and rs[e + 1] == s:
            e += 1
        idx = torch.arange(0, pos[e] + 1)
        blocks = seq_bt[s].long()[idx // bs]
        kk = k_cache[blocks, :, idx % bs, :].float()   # [L, G, D]
        vv = (v_cache[blocks, :, idx % bs, :].float() if v_cache is not None
              else kk[:, :, :V])
        kk = kk.repeat_interleave(rep, dim=1)
        vv = vv.repeat_interleave(rep, dim=1)
        pr = torch.tensor(pos[t:e + 1])
        sc = torch.einsum("ihd,jhd->hij", qf[t:e + 1], kk) * scale
        vis = idx[None, :] <= pr[:, None]
        if window > 0:
            vis &= ((pr[:, None] - idx[None, :] < window)
                    | (idx[None, :] < keep_first))
        sc = sc.masked_fill(~vis[None], float("-inf"))
        m = sc.max(dim=-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink.float().reshape(H, 1, 1))
        ex = torch.exp(sc - m)
        den = ex.sum(dim=-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink.float().reshape(H, 1, 1) - m)
        out[t:e + 1] = torch.einsum("hij,jhd->ihd", ex / den, vv)
        t = e + 1
    if out_gate is not None:
        per_head = out_gate.shape[-1] == H
        out = out * torch.sigmoid(out_gate.float()).reshape(
            T, H, 1 if per_head else V)
    return out.to(q.dtype)


def causal_conv_state(x, conv_w, conv_b, conv_state, seq_cu, seq_slots,
                      positions):
    """Causal convolution over time per channel with a bias: conv_w
    [C, taps] (last column = current token), zeros before the sequence
    start. ``conv_state`` [slots, max(taps-1, 1), C] fp32 keeps each
    sequence's last taps-1 inputs between steps. Returns fp32 [T, C]."""
    T, C = x.shape
    taps = conv_w.shape[1]
    xf = x.float()
    wf = conv_w.float()
    y = torch.empty(T, C, dtype=torch.float32)
    cu, slots, pos = seq_cu.tolist(), seq_slots.tolist(), positions.tolist()
    for s in range(len(slots)):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        slot, p0 = slots[s], pos[a]
        hist = torch.zeros(taps - 1, C, dtype=torch.float32)
        if slot >= 0 and p0 > 0 and taps > 1:
            hist = conv_state[slot, : taps - 1].clone()
        ext = torch.cat([hist, xf[a:b]], dim=0)
        acc = conv_b.float().expand(b - a, C).clone()
        for j in range(taps):
            acc += wf[:, j] * ext[j: j + (b - a)]
        y[a:b] = acc
        if slot >= 0 and taps > 1:
            conv_state[slot, : taps - 1] = ext[-(taps - 1):]
    return y


def rglru_scan(u, gate_lin, gate_bias, lam, y, state, seq_cu, seq_slots,
               positions, decay_scale: float, out_dtype):
    """Real-gated linear recurrence per channel. u [T, W] fp32; gate_lin
    [B, T, 2*bw] fp32 (recurrence gate first, input gate second, W = B*bw)
    plus gate_bias [B, 2*bw]; with r = sigmoid(.), i = sigmoid(.),
    log a = -decay_scale * r * softplus(lam):

        S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t,   out_t = S_t * y_t.

    ``state`` [slots, W] fp32 carries S (zero at position 0)."""
    T, W = u.shape
    B = gate_lin.shape[0]
    bw = W // B
    g = gate_lin.float() + gate_bias.float()[:, None, :]
    r = torch.sigmoid(g[:, :, :bw]).permute(1, 0, 2).reshape(T, W)
    i = torch.sigmoid(g[:, :, bw:]).permute(1, 0, 2).reshape(T, W)
    log_a = -decay_scale * r * torch.nn.functional.softplus(lam.float())
    a = torch.exp(log_a)
    b_in = torch.sqrt(-torch.expm1(2.0 * log_a)) * i * u.float()
    out = torch.empty(T, W, dtype=torch.float32)
    cu, slots, pos = seq_cu.tolist(), seq_slots.tolist(), positions.tolist()
    for s in range(len(slots)):
        t0, t1 = cu[s], cu[s + 1]
        if t1 <= t0:
            continue
        S = _group_state(state, slots[s], pos[t0], (W,))
        for t in range(t0, t1):
            S = a[t] * S + b_in[t]
            out[t] = S
        if slots[s] >= 0:
            state[slots[s]] = S
    return (out * y.float()).to(out_dtype)


def gelu_tanh(x):
    xf = x.float()
    return (0.5 * xf * (1.0 + torch.tanh(
        math.sqrt(2.0 / math.pi) * (xf + 0.044715 * xf.pow(3))))).to(x.dtype)


def relu_squared(x):
    xf = torch.relu(x.float())
    return (xf * xf).to(x.dtype)


# ------------------------------------------------------------------------
# post-norm stream with a token-pair embedding, whole-projection q/k norm
# with blended rotary frequencies, windowed attention that keeps the first
# keys, clamped gated unit, capped logits

def pair_embed(ids, embed, embed_scale: float, pair_table, buckets: int,
               mul_prev: int, mul_cur: int, prev_token, seq_cu, seq_slots,
               positions, act_dtype):
    """x = embed[id] * embed_scale + pair_table[(prev * mul_prev + id *
    mul_cur) mod buckets]; a sequence's first token takes row ``buckets``.
    The previous token of a group's first row comes from ``prev_token``
    [slots] int32, which then receives the group's last id. Returns (fp32
    stream, its rounding to act_dtype). ``pair_table`` None: no pair term."""
    x = embed[ids.long()].float() * embed_scale
    cu = seq_cu.tolist()
    idl = ids.long()
    if pair_table is not None:
        prev = torch.empty_like(idl)
        prev[1:] = idl[:-1]
        first = torch.zeros_like(idl, dtype=torch.bool)
        for s in range(len(cu) - 1):
            a, b = cu[s], cu[s + 1]
            if b <= a:
                continue
            slot = int(seq_slots[s])
            prev[a] = int(prev_token[slot]) if slot >= 0 else 0
            first[a] = True
        row = (prev * mul_prev + idl * mul_cur) % buckets
        row = torch.where(positions.long() == 0,
                          torch.full_like(row, buckets), row)
        x = x + pair_table[row].float()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if b > a and int(seq_slots[s]) >= 0:
            prev_token[int(seq_slots[s])] = int(ids[b - 1])
    return x, x.to(act_dtype)


def layer_norm_affine(x, w, b, eps: float, out_dtype):
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    var = (xf - mu).pow(2).mean(-1, keepdim=True)
    return ((xf - mu) * torch.rsqrt(var + eps) * w.float()
            + b.float()).to(out_dtype)


def post_norm_residual_(resid, y, w, b, eps: float, out_dtype):
    """resid (fp32, in place) += layer_norm(y) * w + b; returns resid
    rounded to out_dtype (the next sublayer's input)."""
    resid += layer_norm_affine(y, w, b, eps, torch.float32)
    return resid.to(out_dtype)


def blended_rotary(dims: int, base: float, factor: float = 1.0,
                   original: float = 0.0, fast: float = 0.0,
                   slow: float = 0.0):
    """([dims/2] fp32 angular frequencies, factor on cos and sin). With
    ``factor`` != 1 every frequency f_i is blended between f_i (pairs that
    turn more than ``fast`` times over ``original`` positions) and
    f_i / factor (fewer than ``slow`` turns), linearly in the pair index
    in between, and cos/sin grow by 0.1 ln(factor) + 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64),
                  -2.0 * i / dims)
    if not original:
        return f.float(), 1.0

    def index_of(turns):
        return (dims * math.log(original / (2.0 * math.pi * turns))
                / (2.0 * math.log(base)))

    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f.float(), 0.1 * math.log(factor) + 1.0


def widenorm_rope_cache_(q, k, v, positions, q_w, k_w, eps: float, inv_freq,
                         rot_mult: float, k_cache, v_cache, slot_mapping,
                         num_heads: int, num_kv_heads: int, dim: int,
                         vdim: int):
    """RMS norm over the WHOLE q row (all heads at once) times q_w, then
    interleaved-pair rotation of the first 2*len(inv_freq) entries of every
    head by p * inv_freq with cos/sin times rot_mult; the same for k, which
    goes into the paged k cache next to the raw v. ``k`` None: only the
    queries (a layer that reads another layer's cache). Returns q
    [T, H, dim]."""
    T = q.shape[0]
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    cos = (torch.cos(ang) * rot_mult)[:, None, :]
    sin = (torch.sin(ang) * rot_mult)[:, None, :]
    nrot = 2 * inv_freq.numel()

    def turn(x, w, heads):
        x = (_rms(x.float(), eps) * w.float()).view(T, heads, dim)
        a, b = x[..., 0:nrot:2], x[..., 1:nrot:2]
        out = x.clone()
        out[..., 0:nrot:2] = a * cos - b * sin
        out[..., 1:nrot:2] = b * cos + a * sin
        return out

    qn = turn(q, q_w, num_heads).to(q.dtype)
    if k is not None:
        kn = turn(k, k_w, num_kv_heads)
        bs = k_cache.shape[2]
        slots = slot_mapping.long()
        ok = slots >= 0
        k_cache[slots[ok] // bs, :, slots[ok] % bs, :] = kn[ok].to(
            k_cache.dtype)
        v_cache[slots[ok] // bs, :, slots[ok] % bs, :] = v.reshape(
            T, num_kv_heads, vdim)[ok].to(v_cache.dtype)
    return qn


def clamped_glu(gu, limit: float):
    """[T, 2F] (gate | up) -> g' sigmoid(1.702 g') (u' + 1) with
    g' = min(g, limit), u' = clamp(u, -limit, limit)."""
    ff = gu.shape[1] // 2
    g = gu[:, :ff].float().clamp(max=limit)
    u = gu[:, ff:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)).to(gu.dtype)


def tanh_cap_(logits, cap: float):
    """logits (fp32, in place) <- cap * tanh(logits / cap)."""
    logits.copy_(cap * torch.tanh(logits / cap))
    return logits

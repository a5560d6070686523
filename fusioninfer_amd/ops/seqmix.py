"""Sequence-mixer ops: scalar-gain RMS norms on an fp32 residual stream,
token shift, shared-key/value rotary attention with chunk/window masks
over the paged cache, the generalized delta rule and its gated output,
and the tanh-GELU gated MLP activation.

Dispatch follows the package policy: GPU tensors run the hand-written
CDNA4 kernels of the ``_C_seqmix`` extension (activations in bf16 or
fp32, statistics/state always fp32) and raise if it is not built; CPU
tensors run the PyTorch implementations in ``seqmix_reference``.

The extension is separate from ``_C`` so that a model that needs only
these ops compiles only these sources on first use.
"""

from __future__ import annotations

from typing import Optional

import torch

from fusioninfer_amd.ops import seqmix_reference as ref

_C = None
_C_ERR: Optional[BaseException] = None


def _load():
    global _C, _C_ERR
    if _C is not None:
        return _C
    try:
        import importlib

        _C = importlib.import_module("fusioninfer_amd.ops._C_seqmix")
    except Exception as e:  # noqa: BLE001 - reported by _native()
        _C_ERR = e
    return _C


def has_native() -> bool:
    return _load() is not None


def _native():
    c = _load()
    if c is None:
        raise RuntimeError(
            "fusioninfer_amd sequence-mixer extension (_C_seqmix.so) is not "
            "available but a GPU tensor was passed; build it with "
            "`python -m fusioninfer_amd.ops.build seqmix`."
        ) from _C_ERR
    return c


def scalar_rms_norm(x, g, eps: float, out_dtype):
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _native().scalar_rms_norm(out, x, g, eps)
        return out
    return ref.scalar_rms_norm(x, g, eps, out_dtype)


def residual_add_scalar_norm_(resid, y, g_post, eps: float, g_next=None,
                              out_dtype=None):
    if resid.is_cuda:
        out = None
        if g_next is not None:
            out = torch.empty(resid.shape, dtype=out_dtype,
                              device=resid.device)
        _native().residual_add_scalar_norm(resid, y, g_post, g_next, out, eps)
        return out
    return ref.residual_add_scalar_norm_(resid, y, g_post, eps, g_next,
                                         out_dtype)


def norm_token_shift(resid, g, shift, state, seq_cu, row_seq, positions,
                     seq_slots, eps: float, out_dtype):
    if resid.is_cuda:
        out = torch.empty(resid.shape, dtype=out_dtype, device=resid.device)
        _native().norm_token_shift(out, resid, g, shift, state, seq_cu,
                                   row_seq, positions, seq_slots, eps)
        return out
    return ref.norm_token_shift(resid, g, shift, state, seq_cu, row_seq,
                                positions, seq_slots, eps, out_dtype)


def rope_unitnorm_cache_(q, k, positions, inv_freq, eps: float, k_cache,
                         v_cache, slot_mapping, num_heads: int,
                         num_kv_heads: int, head_dim: int):
    """q/k may be column slices of one projection output (row stride >
    width); returns a fresh contiguous processed q [T, H, D]."""
    if q.is_cuda:
        T = q.shape[0]
        out = torch.empty((T, num_heads, head_dim), dtype=q.dtype,
                          device=q.device)
        _native().rope_unitnorm_cache(out, q, k, positions, inv_freq,
                                      k_cache, v_cache, slot_mapping,
                                      num_heads, num_kv_heads, head_dim, eps)
        return out
    return ref.rope_unitnorm_cache_(q, k, positions, inv_freq, eps, k_cache,
                                    v_cache, slot_mapping, num_heads,
                                    num_kv_heads, head_dim)


ATTENTION_TILE_ROWS = 128  # q rows per workgroup of the tiled kernel


def build_attention_tiles(group_lens, device=None):
    """Tile table of the tiled attention kernel: one entry per
    ATTENTION_TILE_ROWS rows of every row group, (group, first row inside
    the group). Returns (tile_seq, tile_row0, rows covered)."""
    tile_seq, tile_row0 = [], []
    for s, n in enumerate(group_lens):
        for r0 in range(0, n, ATTENTION_TILE_ROWS):
            tile_seq.append(s)
            tile_row0.append(r0)
    return (torch.tensor(tile_seq, dtype=torch.int32, device=device),
            torch.tensor(tile_row0, dtype=torch.int32, device=device),
            int(sum(group_lens)))


def ranged_paged_attention(q, k_cache, v_cache, seq_bt, row_seq, positions,
                           scale: float, chunk: int = 0, window: int = 0,
                           seq_cu=None, tiles=None):
    """``tiles`` = build_attention_tiles(lens of the LEADING row groups):
    on the GPU those rows run the tiled MFMA kernel (prompt portions), the
    remaining rows (one-row decode groups) the row-per-wave kernel."""
    if q.is_cuda:
        T, H, D = q.shape
        out = torch.empty((T, H, v_cache.shape[3]), dtype=q.dtype,
                          device=q.device)
        tile_seq = tile_row0 = None
        tile_rows = 0
        if tiles is not None and seq_cu is not None and tiles[2] > 0:
            tile_seq, tile_row0, tile_rows = tiles
        _native().ranged_paged_attention(out, q, k_cache, v_cache, seq_bt,
                                         row_seq, positions, scale,
                                         int(chunk), int(window), seq_cu,
                                         tile_seq, tile_row0, int(tile_rows))
        return out
    return ref.ranged_paged_attention(q, k_cache, v_cache, seq_bt, row_seq,
                                      positions, scale, chunk, window)


def delta_rule(r, k, v, wlin, alin, glin, w0, a_bias, norm_w, state,
               seq_cu, seq_slots, positions, heads: int, dim: int,
               eps: float, decay_scale: float):
    if r.is_cuda:
        T = r.shape[0]
        out = torch.empty((T, heads * dim), dtype=r.dtype, device=r.device)
        o_raw = torch.empty((T, heads * dim), dtype=torch.float32,
                            device=r.device)
        # scratch for the state-independent per-token vectors; the last
        # dim is the kernel's row capacity for this head size
        cap = 64 if dim <= 64 else (128 if dim <= 128 else 256)
        vecs = torch.empty((T, heads, 5, cap), dtype=torch.float32,
                           device=r.device)
        _native().delta_rule(out, o_raw, vecs, r, k, v, wlin, alin, glin, w0, a_bias,
                             norm_w, state, seq_cu, seq_slots, positions,
                             heads, dim, eps, decay_scale)
        return out
    return ref.delta_rule(r, k, v, wlin, alin, glin, w0, a_bias, norm_w,
                          state, seq_cu, seq_slots, positions, heads, dim,
                          eps, decay_scale)


def dual_norm_combine_residual_(resid, yl, yr, wl, wr, g_post, eps: float,
                                g_next=None, out_dtype=None):
    if resid.is_cuda:
        out = None
        if g_next is not None:
            out = torch.empty(resid.shape, dtype=out_dtype,
                              device=resid.device)
        _native().dual_norm_combine_residual(resid, yl, yr, wl, wr, g_post,
                                             g_next, out, eps)
        return out
    return ref.dual_norm_combine_residual_(resid, yl, yr, wl, wr, g_post,
                                           eps, g_next, out_dtype)


def gelu_tanh_and_mul(gu):
    if gu.is_cuda:
        out = torch.empty((gu.shape[0], gu.shape[1] // 2), dtype=gu.dtype,
                          device=gu.device)
        _native().gelu_tanh_and_mul(out, gu)
        return out
    return ref.gelu_tanh_and_mul(gu)


# ------------------------------------------------------------------------
# layer-norm / gated-residual stream, decayed linear attention, windowed
# attention with head mixing, gated delta rule

def layer_norm(x, w, eps: float, out_dtype):
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _native().layer_norm(out, x, w, eps)
        return out
    return ref.layer_norm(x, w, eps, out_dtype)


def gated_residual_layer_norm_(resid, y1, s1: float, y2, s2: float, gate_lin,
                               gate_bias, w_next, eps: float, out_dtype):
    """resid (fp32, in place) += (s1*y1 + s2*y2) * sigmoid(gate_lin +
    gate_bias); returns layer_norm(resid) * w_next (None without w_next).
    gate_lin may be a column slice of a wider projection output."""
    if resid.is_cuda:
        out = None
        if w_next is not None:
            out = torch.empty(resid.shape, dtype=out_dtype,
                              device=resid.device)
        _native().gated_residual_layer_norm(resid, y1, float(s1), y2,
                                            float(s2), gate_lin, gate_bias,
                                            w_next, out, eps)
        return out
    return ref.gated_residual_layer_norm_(resid, y1, s1, y2, s2, gate_lin,
                                          gate_bias, w_next, eps, out_dtype)


def _recurrence_scratch(T: int, heads: int, dim: int, device):
    """fp32 scratch of the recurrence kernel: five vectors per (token,
    head), padded to the kernel's row capacity for this key size."""
    if dim > 256:
        raise ValueError("recurrent mixers support key sizes up to 256")
    cap = 64 if dim <= 64 else (128 if dim <= 128 else 256)
    return torch.empty((T, heads, 5, cap), dtype=torch.float32,
                       device=device)


def decay_linear_attention(q, k, v, decay, state, seq_cu, seq_slots,
                           positions, heads: int, dim: int, vdim: int,
                           silu: bool = True, row_seq=None):
    """Raw fp32 read-outs [T, heads*vdim] of linear attention with one
    scalar decay per head; q/k/v may be column slices of one projection
    output. With ``row_seq`` (group of every row) the GPU path runs
    multi-row groups through the chunk-parallel kernel."""
    if q.is_cuda:
        T = q.shape[0]
        o_raw = torch.empty((T, heads * vdim), dtype=torch.float32,
                            device=q.device)
        vecs = _recurrence_scratch(T, heads, dim, q.device)
        vbuf = torch.empty((T, heads * vdim), dtype=torch.float32,
                           device=q.device)
        _native().decay_linear_attention(o_raw, vecs, vbuf, q, k, v, decay,
                                         state, seq_cu, seq_slots, positions,
                                         heads, dim, vdim, bool(silu),
                                         row_seq)
        return o_raw
    return ref.decay_linear_attention(q, k, v, decay, state, seq_cu,
                                      seq_slots, positions, heads, dim, vdim,
                                      silu)


def group_rms_gate(o_raw, glin, w, groups: int, eps: float, gate: str,
                   out_dtype):
    if gate not in ("sigmoid", "silu"):
        raise ValueError(f"unknown gate {gate!r}")
    if o_raw.is_cuda:
        out = torch.empty(o_raw.shape, dtype=out_dtype, device=o_raw.device)
        _native().group_rms_gate(out, o_raw, glin, w, int(groups), eps,
                                 gate == "silu")
        return out
    return ref.group_rms_gate(o_raw, glin, w, groups, eps, gate, out_dtype)


def paged_cache_write_(k, v, k_cache, v_cache, slot_mapping):
    if k.is_cuda:
        _native().paged_cache_write(k, v, k_cache, v_cache, slot_mapping)
        return
    ref.paged_cache_write_(k, v, k_cache, v_cache, slot_mapping)


def talking_window_attention(q, k_cache, v_cache, seq_bt, row_seq, positions,
                             scale: float, window: int, r1, r2, talk,
                             heads: int, seq_cu=None, tiles=None):
    """q: [T, heads*dim] (may be a column slice); returns [T, heads, vdim].
    ``tiles`` as for ranged_paged_attention: the leading row groups that
    are prompt portions."""
    T = q.shape[0]
    dim = q.shape[1] // heads
    if q.is_cuda:
        out = torch.empty((T, heads, v_cache.shape[3]), dtype=q.dtype,
                          device=q.device)
        tile_seq = tile_row0 = folded = pen = None
        tile_rows = 0
        if tiles is not None and seq_cu is not None and tiles[2] > 0:
            tile_seq, tile_row0, tile_rows = tiles
            # scratch of the tiled kernel: queries with the head mixing
            # folded in (one segment per kv head) and the mixed distance
            # penalty for every distance a row can reach
            G, bs = k_cache.shape[1], k_cache.shape[2]
            folded = torch.empty((tile_rows, heads, G, dim), dtype=q.dtype,
                                 device=q.device)
            maxd = int(window) if window > 0 else seq_bt.shape[1] * bs
            pen = torch.empty((heads, maxd), dtype=torch.float32,
                              device=q.device)
        part_ml = part_o = None
        rest = T - tile_rows
        if rest > 0:
            # rows outside the tile table (decoded rows): one partial
            # result per 256-key pass of the visible range
            bs = k_cache.shape[2]
            keys = int(window) if window > 0 else seq_bt.shape[1] * bs
            ns = _native().talking_window_splits(keys)
            V = v_cache.shape[3]
            part_ml = torch.empty((rest, ns, 2, heads), dtype=torch.float32,
                                  device=q.device)
            part_o = torch.empty((rest, ns, heads * V), dtype=torch.float32,
                                 device=q.device)
        _native().talking_window_attention(out, q, k_cache, v_cache, seq_bt,
                                           row_seq, positions, float(scale),
                                           int(window), r1, r2, talk,
                                           int(heads), seq_cu, tile_seq,
                                           tile_row0, int(tile_rows), folded,
                                           pen, part_ml, part_o)
        return out
    return ref.talking_window_attention(
        q.reshape(T, heads, dim), k_cache, v_cache, seq_bt, row_seq,
        positions, scale, window, r1, r2, talk)


def gated_delta_rule(x, conv_w, alin, blin, a_log, dt_bias, conv_state,
                     state, seq_cu, seq_slots, positions, heads: int,
                     kv_heads: int, dim: int, vdim: int, row_seq=None):
    """Raw fp32 read-outs [T, heads*vdim] of the gated delta rule behind a
    short causal convolution; x = q|k|v projections [T, C] (row-strided)."""
    if x.is_cuda:
        T = x.shape[0]
        o_raw = torch.empty((T, heads * vdim), dtype=torch.float32,
                            device=x.device)
        vecs = _recurrence_scratch(T, heads, dim, x.device)
        vbuf = torch.empty((T, heads * vdim), dtype=torch.float32,
                           device=x.device)
        _native().gated_delta_rule(o_raw, vecs, vbuf, x, conv_w, alin, blin,
                                   a_log, dt_bias, conv_state, state, seq_cu,
                                   seq_slots, positions, row_seq, heads,
                                   kv_heads, dim, vdim)
        return o_raw
    return ref.gated_delta_rule(x, conv_w, alin, blin, a_log, dt_bias,
                                conv_state, state, seq_cu, seq_slots,
                                positions, heads, kv_heads, dim, vdim)


# ------------------------------------------------------------------------
# parallel-residual stream, weighted head norms with a query temperature,
# latent keys/values with a softmax sink, gated linear recurrence

def scaled_residual_layer_norm_(resid, ys, scales, w_next, eps: float,
                                out_dtype):
    """resid (fp32, in place) += sum_i scales[i] * ys[i] for one to three
    sublayer results; returns layer_norm(resid) * w_next (None without
    w_next)."""
    if not 1 <= len(ys) <= 3 or len(ys) != len(scales):
        raise ValueError("one to three terms, one scale each")
    if resid.is_cuda:
        out = None
        if w_next is not None:
            out = torch.empty(resid.shape, dtype=out_dtype,
                              device=resid.device)
        ys = list(ys) + [None] * (3 - len(ys))
        sc = [float(s) for s in scales] + [0.0] * (3 - len(scales))
        _native().scaled_residual_layer_norm(resid, ys[0], sc[0], ys[1],
                                             sc[1], ys[2], sc[2], w_next,
                                             out, eps)
        return out
    return ref.scaled_residual_layer_norm_(resid, ys, scales, w_next, eps,
                                           out_dtype)


def cast_layer_norm(y, w_next, eps: float):
    """Restart the fp32 stream from the activation rows y: returns (fp32
    copy of y, layer_norm of it times w_next in y's dtype or None)."""
    if y.is_cuda:
        resid = torch.empty(y.shape, dtype=torch.float32, device=y.device)
        out = torch.empty_like(y) if w_next is not None else None
        _native().cast_layer_norm(resid, out, y, w_next, eps)
        return resid, out
    return ref.cast_layer_norm(y, w_next, eps)


def concat_cast(resid, x0):
    """[resid rounded to x0's dtype | x0]: input rows of a product that
    reads the stream next to an activation."""
    if resid.is_cuda:
        out = torch.empty((resid.shape[0], 2 * resid.shape[1]),
                          dtype=x0.dtype, device=x0.device)
        _native().concat_cast(out, resid, x0)
        return out
    return ref.concat_cast(resid, x0)


def headnorm_qtemp_cache_(q, k, v, positions, q_w, k_w, eps: float,
                          temp_coef: float, temp_every: int, k_cache,
                          v_cache, slot_mapping, num_heads: int,
                          num_kv_heads: int, dim: int, vdim: int):
    """q/k/v may be column slices of one projection output; returns a
    fresh contiguous processed q [T, H, dim]."""
    if q.is_cuda:
        out = torch.empty((q.shape[0], num_heads, dim), dtype=q.dtype,
                          device=q.device)
        _native().headnorm_qtemp_cache(out, q, k, v, positions, q_w, k_w,
                                       eps, float(temp_coef),
                                       int(temp_every), k_cache, v_cache,
                                       slot_mapping, num_heads,
                                       num_kv_heads, dim, vdim)
        return out
    return ref.headnorm_qtemp_cache_(q, k, v, positions, q_w, k_w, eps,
                                     temp_coef, temp_every, k_cache, v_cache,
                                     slot_mapping, num_heads, num_kv_heads,
                                     dim, vdim)


def latent_rope_cache_(q, ckr, positions, inv_freq, norm_w, eps: float,
                       kv_cache, slot_mapping, num_heads: int, dim: int,
                       rot_dim: int, rank: int, q_out):
    """Writes the rotated query parts into q_out[:, :, rank:] ([T, H,
    rank+rot_dim]) and the normed latent + rotated shared key part into
    the paged cache."""
    if q.is_cuda:
        _native().latent_rope_cache(q_out, q, ckr, positions, inv_freq,
                                    norm_w, eps, kv_cache, slot_mapping,
                                    num_heads, dim, rot_dim, rank)
        return
    ref.latent_rope_cache_(q, ckr, positions, inv_freq, norm_w, eps,
                           kv_cache, slot_mapping, num_heads, dim, rot_dim,
                           rank, q_out)


SPLIT_ROWS_PER_LAUNCH = 512  # rows per launch of the split attention form


def sink_paged_attention(q, k_cache, v_cache, seq_bt, row_seq, positions,
                         scale: float, sink=None, value_dims: int = 0,
                         out_gate=None, seq_cu=None, tiles=None,
                         window: int = 0, keep_first: int = 0):
    """Causal softmax attention over the paged cache with separate key and
    value sizes, an optional per-head sink in the denominator, values that
    may be the leading ``value_dims`` entries of the cached keys
    (``v_cache`` None) and an optional sigmoid gate on the result, per
    (row, head) ([T, H]) or per entry ([T, H*Dv]). ``window`` > 0 hides
    key j from position p unless p - j < window or j < keep_first.
    ``tiles`` as for ranged_paged_attention."""
    if q.is_cuda:
        T, H, _ = q.shape
        V = v_cache.shape[3] if v_cache is not None else int(value_dims)
        out = torch.empty((T, H, V), dtype=q.dtype, device=q.device)
        tile_seq = tile_row0 = None
        tile_rows = 0
        if (tiles is not None and seq_cu is not None and tiles[2] > 0
                and _native().sink_attention_has_tiles(q.shape[2], V)):
            tile_seq, tile_row0, tile_rows = tiles
        rest = T - tile_rows
        part_ml = part_o = None
        if rest > 0:
            # rows outside the tile table: partial results per span of the
            # cache capacity, at most SPLIT_ROWS_PER_LAUNCH rows at a time
            bs = k_cache.shape[2]
            ns = _native().sink_attention_splits(seq_bt.shape[1] * bs)
            cap = min(rest, SPLIT_ROWS_PER_LAUNCH)
            part_ml = torch.empty((cap, H, ns, 2), dtype=torch.float32,
                                  device=q.device)
            part_o = torch.empty((cap, H, ns, V), dtype=torch.float32,
                                 device=q.device)
        _native().sink_paged_attention(out, q, k_cache, v_cache, seq_bt,
                                       row_seq, positions, float(scale),
                                       sink, V, out_gate, seq_cu, tile_seq,
                                       tile_row0, int(tile_rows), part_ml,
                                       part_o, int(window), int(keep_first))
        return out
    return ref.sink_paged_attention(q, k_cache, v_cache, seq_bt, row_seq,
                                    positions, scale, sink, value_dims,
                                    out_gate, window, keep_first)


def causal_conv_state(x, conv_w, conv_b, conv_state, seq_cu, row_seq,
                      seq_slots, positions):
    """fp32 [T, C] causal convolution of x (a column slice is fine) with
    the per-sequence tail kept in conv_state."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        _native().causal_conv_state(out, x, conv_w, conv_b, conv_state,
                                    seq_cu, row_seq, seq_slots, positions)
        return out
    return ref.causal_conv_state(x, conv_w, conv_b, conv_state, seq_cu,
                                 seq_slots, positions)


def rglru_scan(u, gate_lin, gate_bias, lam, y_lin, state, seq_cu, seq_slots,
               positions, decay_scale: float, out_dtype, max_rows: int = 0):
    """Gated linear recurrence over the rows of every group; returns
    S_t * gelu_tanh(y_lin_t) in out_dtype. ``max_rows``: longest group of
    the step (0: unknown)."""
    if u.is_cuda:
        out = torch.empty(u.shape, dtype=out_dtype, device=u.device)
        _native().rglru_scan(out, u, gate_lin, gate_bias, lam, y_lin, state,
                             seq_cu, seq_slots, positions,
                             float(decay_scale), int(max_rows))
        return out
    return ref.rglru_scan(u, gate_lin, gate_bias, lam,
                          ref.gelu_tanh(y_lin.float()), state, seq_cu,
                          seq_slots, positions, decay_scale, out_dtype)


def relu_squared(x):
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _native().relu_squared(out, x)
        return out
    return ref.relu_squared(x)


# ------------------------------------------------------------------------
# post-norm stream with a token-pair embedding, whole-projection q/k norm
# with blended rotary frequencies, clamped gated unit, capped logits

blended_rotary = ref.blended_rotary


def pair_embed(ids, embed, embed_scale: float, pair_table, buckets: int,
               mul_prev: int, mul_cur: int, prev_token, seq_cu, row_seq,
               seq_slots, positions, act_dtype):
    """Start of an fp32 stream: embed[id] * embed_scale plus the pair
    table's row for (previous id, id) (row ``buckets`` at position 0). The
    previous id of a group's first row is read from ``prev_token`` [slots]
    int32, which then receives the group's last id. Returns (fp32 stream,
    its rounding to act_dtype)."""
    if embed.is_cuda:
        T, W = ids.shape[0], embed.shape[1]
        resid = torch.empty((T, W), dtype=torch.float32, device=embed.device)
        act = (resid if act_dtype == torch.float32 else
               torch.empty((T, W), dtype=act_dtype, device=embed.device))
        _native().pair_embed(resid, act, ids, embed, float(embed_scale),
                             pair_table, int(buckets), int(mul_prev),
                             int(mul_cur), prev_token, seq_cu, row_seq,
                             seq_slots, positions)
        return resid, act
    return ref.pair_embed(ids, embed, embed_scale, pair_table, buckets,
                          mul_prev, mul_cur, prev_token, seq_cu, seq_slots,
                          positions, act_dtype)


def layer_norm_affine(x, w, b, eps: float, out_dtype):
    """(x - mean) / sqrt(var + eps) * w + b with fp32 statistics."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _native().layer_norm_affine(out, x, w, b, eps)
        return out
    return ref.layer_norm_affine(x, w, b, eps, out_dtype)


def post_norm_residual_(resid, y, w, b, eps: float, out_dtype):
    """resid (fp32, in place) += layer_norm(y) * w + b, the norm sitting on
    the sublayer's OUTPUT y; returns resid rounded to out_dtype (resid
    itself for fp32), the next sublayer's input."""
    if resid.is_cuda:
        out = (resid if out_dtype == torch.float32 else
               torch.empty(resid.shape, dtype=out_dtype, device=resid.device))
        _native().post_norm_residual(resid, y, w, b, out, eps)
        return out
    return ref.post_norm_residual_(resid, y, w, b, eps, out_dtype)


def widenorm_rope_cache_(q, k, v, positions, q_w, k_w, eps: float, inv_freq,
                         rot_mult: float, k_cache, v_cache, slot_mapping,
                         num_heads: int, num_kv_heads: int, dim: int,
                         vdim: int):
    """RMS norm over the whole q (and k) row times a weight vector, then
    interleaved-pair rotation of the leading 2*len(inv_freq) entries of
    every head (cos/sin times rot_mult); processed k and raw v go into the
    paged caches. ``k`` None: queries only. q/k/v may be column slices of
    one projection output; returns a fresh contiguous q [T, H, dim]."""
    if q.is_cuda:
        out = torch.empty((q.shape[0], num_heads, dim), dtype=q.dtype,
                          device=q.device)
        _native().widenorm_rope_cache(out, q, k, v, positions, q_w, k_w, eps,
                                      inv_freq, float(rot_mult), k_cache,
                                      v_cache, slot_mapping, num_heads,
                                      num_kv_heads, dim, vdim)
        return out
    return ref.widenorm_rope_cache_(q, k, v, positions, q_w, k_w, eps,
                                    inv_freq, rot_mult, k_cache, v_cache,
                                    slot_mapping, num_heads, num_kv_heads,
                                    dim, vdim)


def clamped_glu(gu, limit: float):
    """[T, 2F] (gate | up) -> [T, F]: g' sigmoid(1.702 g') (u' + 1) with
    g' = min(g, limit), u' = clamp(u, -limit, limit)."""
    if gu.is_cuda:
        out = torch.empty((gu.shape[0], gu.shape[1] // 2), dtype=gu.dtype,
                          device=gu.device)
        _native().clamped_glu(out, gu, float(limit))
        return out
    return ref.clamped_glu(gu, limit)


def tanh_cap_(logits, cap: float):
    """fp32 logits, in place: cap * tanh(logits / cap)."""
    if logits.is_cuda:
        _native().tanh_cap(logits, float(cap))
        return logits
    return ref.tanh_cap_(logits, cap)

"""Sequence-mixer building blocks beyond plain causal softmax attention.

Each block is a mechanism with its constants as constructor parameters, so
model designs assemble them freely:

* ``SharedKVAttention``  rotary attention whose values ARE the projected
  keys (no value projection), interleaved-pair partial rotary, unit-RMS
  q/k, explicit score scale, chunk and/or sliding-window masks; reads and
  writes the engine's paged cache.
* ``DeltaRuleMixer``     generalized delta rule (per-channel decay from a
  low-rank branch, per-channel removal rate), fp32 recurrent state kept in
  the engine's state slots, per-head unit-RMS output with gain and gate.
* ``ParallelMixer``      two mixers side by side on one input with ONE
  merged input projection; the halves are width-normalized and averaged by
  the caller's fused residual kernel.
* ``GatedMLP``           act(gate) * up -> down with a chosen activation.
* ``DecayLinearAttention``  linear attention with one scalar decay per
  head (silu feature maps), fp32 state in the state slots, whole-row
  unit-RMS output with gain and sigmoid gate.
* ``TalkingWindowAttention``  grouped-query softmax attention without
  rotation: projection biases, a log-distance score penalty per head,
  scores mixed across heads before the softmax, sliding window; separate
  key and value sizes in the paged cache.
* ``GatedDeltaMixer``    gated delta rule (scalar decay and write strength
  per head and token) behind a short causal convolution whose tail is
  part of the slot state; per-head unit-RMS output with a shared gain and
  a silu gate.
* ``RoutedExperts``      mixture of gated feed-forward experts with a
  sigmoid or softmax router, top-k choice, optional renormalisation and a
  constant factor on the weights.
* ``TemperedGatedAttention``  grouped-query softmax attention without
  rotation: projection biases, a weighted RMS norm per query/key head, a
  query factor that grows with the logarithm of the position's block
  index, and a sigmoid gate per head on the result.
* ``LatentAttention``    keys and values expanded from one normed low-rank
  latent per token plus one rotated key part shared by all heads; only the
  latent and the rotated part are cached, the expansions are folded into
  the queries and the attended latents; optional per-head softmax sink.
* ``RGLRUMixer``         real-gated linear recurrent unit behind a short
  causal convolution with block-diagonal gates, times a GELU branch.
* ``SquaredReluMLP``     down(relu(up x)^2) whose up projection may ride a
  layer's merged input projection.
* ``ParallelResidualLayer`` one layer norm feeding a mixer and a
  feed-forward side by side, x <- x + m (mixer + ff), all input branches
  in ONE merged projection.
* ``GatedResidualLayer`` layer-normed residual layer whose sublayer
  results are multiplied by sigmoid(W h + b) before they are added; one
  mixer or several scaled mixers side by side behind ONE merged input
  projection (which also carries the gate's W).

* ``WindowedSinkAttention``  grouped-query softmax attention with
  projection biases, ONE RMS norm over the whole query (and key)
  projection, interleaved partial rotary positions whose frequencies can
  be blended for context extension, a sliding window that always keeps the
  first keys, a per-head softmax sink and an elementwise sigmoid gate; a
  layer may read another layer's paged keys and values instead of
  projecting its own.
* ``ClampedGatedMLP``    down(g' sigmoid(1.702 g') (u' + 1)) with the gate
  clamped from above and the up branch on both sides.
* ``PostNormLayer``      x <- x + LN(mixer(x)), x <- x + LN(ff(x)): the
  sublayers read the stream itself and the layer norm (weight and bias)
  sits on their output.

Activations run in the model dtype (bf16 or fp32); statistics, rotary
angles, scores, decays, gates of the recurrence and the state are fp32
inside the ops (fusioninfer_amd/ops/seqmix.py).
"""

from __future__ import annotations

import dataclasses
import math
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from fusioninfer_amd.distributed.layers import (
    MergedColumnParallelLinear,
    ReplicatedLinear,
    RowParallelLinear,
)
from fusioninfer_amd.ops import seqmix


@dataclasses.dataclass
class SharedKVAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                 # per-head query/key size
    vdim: int                # per-head value size (== dim: values are keys)
    scale: float             # score multiplier
    rot_dims: int            # leading dims of each head that rotate
    rot_base: float
    chunk: int = 0           # >0: keys only from the query's own chunk
    window: int = 0          # >0: keys only from the last `window` positions

    def __post_init__(self):
        if self.vdim != self.dim:
            raise ValueError(
                "shared key/value attention needs vdim == dim "
                f"(got dim={self.dim}, vdim={self.vdim})")
        if self.heads % self.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if self.rot_dims % 2 or not 0 <= self.rot_dims <= self.dim:
            raise ValueError("rot.dims must be even and <= dim")


@dataclasses.dataclass
class DeltaRuleConfig:
    heads: int
    dim: int                 # per-head key = value size
    decay_rank: int          # inner size of the low-rank decay branch
    # decay w = exp(-decay_scale * sigmoid(.)): the design's fixed constant
    decay_scale: float = math.exp(-0.5)


def _f32_param(shape, fill: float = 1.0) -> nn.Parameter:
    """Small gains/biases stay fp32 whatever the model dtype (they enter
    32-bit statistics only)."""
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32),
                        requires_grad=False)


def rotary_inv_freq(dims: int, base: float) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2, rounded once to fp32 (angles are
    position * f_i in fp32)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / max(dims, 1))).to(torch.float32)


class SharedKVAttention(nn.Module):
    """Attention half: consumes its slice of the merged projection."""

    def __init__(self, cfg: SharedKVAttentionConfig, width: int, eps: float,
                 dtype):
        super().__init__()
        self.cfg = cfg
        self.eps = eps
        self.q_size = cfg.heads * cfg.dim
        self.k_size = cfg.kv_heads * cfg.dim
        self.in_sizes = [self.q_size, self.k_size]
        self.in_names = ["q", "k"]
        self.o_proj = RowParallelLinear(cfg.heads * cfg.vdim, width,
                                        dtype=dtype)
        self.register_buffer(
            "inv_freq", rotary_inv_freq(cfg.rot_dims, cfg.rot_base),
            persistent=False)

    def cache_shape(self, num_blocks: int, block_size: int):
        c = self.cfg
        return (num_blocks, c.kv_heads, block_size, c.dim)

    def forward(self, parts, meta, cache) -> torch.Tensor:
        q, k = parts
        c = self.cfg
        k_cache, v_cache = cache["k"], cache["v"]
        qn = seqmix.rope_unitnorm_cache_(
            q, k, meta.positions, self.inv_freq, self.eps, k_cache, v_cache,
            meta.slot_mapping, c.heads, c.kv_heads, c.dim)
        o = seqmix.ranged_paged_attention(
            qn, k_cache, v_cache, meta.seq_bt, meta.row_seq, meta.positions,
            c.scale, chunk=c.chunk, window=c.window, seq_cu=meta.seq_cu,
            tiles=meta.seq_tiles)
        return self.o_proj(o.view(o.shape[0], c.heads * c.vdim))


class DeltaRuleMixer(nn.Module):
    """Recurrent half: r/k/v/gate/removal/decay branches come from the
    merged projection; the decay branch is low-rank (tanh between)."""

    def __init__(self, cfg: DeltaRuleConfig, width: int, eps: float, dtype):
        super().__init__()
        self.cfg = cfg
        self.eps = eps
        n = cfg.heads * cfg.dim
        self.in_sizes = [n, n, n, n, n, cfg.decay_rank]
        self.in_names = ["r", "k", "v", "g", "a", "w1"]
        self.w2 = ReplicatedLinear(cfg.decay_rank, n, dtype=dtype)
        self.w0 = _f32_param((n,), 0.0)
        self.a_bias = _f32_param((n,), 0.0)
        self.norm_w = _f32_param((n,), 1.0)
        self.o_proj = RowParallelLinear(n, width, dtype=dtype)

    def state_shape(self):
        c = self.cfg
        return (c.heads, c.dim, c.dim)

    def forward(self, parts, meta, cache) -> torch.Tensor:
        r, k, v, g, a, w1 = parts
        c = self.cfg
        wlin = self.w2(torch.tanh(w1))
        o = seqmix.delta_rule(
            r, k, v, wlin, a, g, self.w0, self.a_bias, self.norm_w,
            cache["delta"], meta.seq_cu, meta.seq_slots, meta.positions,
            c.heads, c.dim, self.eps, c.decay_scale)
        return self.o_proj(o)


class ParallelMixer(nn.Module):
    """Two mixers reading the same input through one merged GEMM. Returns
    both halves' projected outputs and their width gains; the caller's
    fused kernel normalizes, averages and adds them to the residual."""

    def __init__(self, left: nn.Module, right: nn.Module, width: int, dtype):
        super().__init__()
        self.left = left
        self.right = right
        self.sizes: List[int] = list(left.in_sizes) + list(right.in_sizes)
        self.n_left = len(left.in_sizes)
        self.in_proj = MergedColumnParallelLinear(width, self.sizes,
                                                  dtype=dtype)
        self.left_out = _f32_param((width,), 1.0)
        self.right_out = _f32_param((width,), 1.0)

    def in_proj_rows(self, side: str, name: str):
        """(row offset, rows) of a named branch inside the merged weight."""
        names = [("left", n) for n in self.left.in_names] + \
                [("right", n) for n in self.right.in_names]
        off = 0
        for (s, n), size in zip(names, self.sizes):
            if (s, n) == (side, name):
                return off, size
            off += size
        raise KeyError((side, name))

    def forward(self, h, meta, cache):
        parts = self.in_proj(h).split(self.sizes, dim=-1)
        yl = self.left(parts[: self.n_left], meta, cache)
        yr = self.right(parts[self.n_left:], meta, cache)
        return yl, yr


class GatedMLP(nn.Module):
    """down(act(gate(x)) * up(x)); ``act`` names the fused activation."""

    def __init__(self, width: int, ff: int, dtype, act: str = "gelu_tanh"):
        super().__init__()
        if act != "gelu_tanh":
            raise ValueError(f"unsupported gated-MLP activation {act!r}")
        self.gate_up_proj = MergedColumnParallelLinear(width, [ff, ff],
                                                       dtype=dtype)
        self.down_proj = RowParallelLinear(ff, width, dtype=dtype)

    def forward(self, x):
        return self.down_proj(seqmix.gelu_tanh_and_mul(self.gate_up_proj(x)))


class MixerLayer(nn.Module):
    """Pre- and post-normed residual layer on an fp32 stream with
    scalar-gain RMS norms and a token shift in front of the mixer:

        x <- x + norm1b(mixer(shift(norm1(x))));  x <- x + norm2b(ff(norm2(x)))
    """

    def __init__(self, mixer: ParallelMixer, mlp: Optional[GatedMLP],
                 width: int, eps: float, dtype):
        super().__init__()
        self.mixer = mixer
        self.mlp = mlp
        self.eps = eps
        self.dtype = dtype
        self.norm1 = _f32_param((1,))
        self.norm1b = _f32_param((1,))
        self.norm2 = _f32_param((1,)) if mlp is not None else None
        self.norm2b = _f32_param((1,)) if mlp is not None else None
        self.shift = _f32_param((width,), 0.0)

    def forward(self, resid, meta, cache):
        h = seqmix.norm_token_shift(
            resid, self.norm1, self.shift, cache["shift"], meta.seq_cu,
            meta.row_seq, meta.positions, meta.seq_slots, self.eps,
            self.dtype)
        yl, yr = self.mixer(h, meta, cache)
        h2 = seqmix.dual_norm_combine_residual_(
            resid, yl, yr, self.mixer.left_out, self.mixer.right_out,
            self.norm1b, self.eps, self.norm2, self.dtype)
        if self.mlp is not None:
            seqmix.residual_add_scalar_norm_(
                resid, self.mlp(h2), self.norm2b, self.eps)
        return resid


# ------------------------------------------------------------------------
# Layer-norm / gated-residual family of blocks


@dataclasses.dataclass
class DecayLinearAttentionConfig:
    heads: int
    dim: int                 # per-head query/key size
    vdim: int                # per-head value size
    decay: Tuple[float, ...]  # one factor per head

    def __post_init__(self):
        if len(self.decay) != self.heads:
            raise ValueError("one decay per head is needed "
                             f"(got {len(self.decay)} for {self.heads})")


@dataclasses.dataclass
class TalkingWindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0          # >0: keys only from the last `window` positions

    def __post_init__(self):
        if self.heads % self.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")


@dataclasses.dataclass
class GatedDeltaConfig:
    heads: int               # value heads (= state heads)
    kv_heads: int            # query/key heads
    dim: int
    vdim: int
    conv: int                # taps of the causal convolution (1 = none)

    def __post_init__(self):
        if self.heads % self.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if self.conv < 1:
            raise ValueError("conv taps must be >= 1")


def _f32_rand(shape, lo: float, hi: float) -> nn.Parameter:
    return nn.Parameter(
        torch.rand(shape, dtype=torch.float32) * (hi - lo) + lo,
        requires_grad=False)


class DecayLinearAttention(nn.Module):
    """Linear-attention mixer: consumes its slice of the merged projection
    (q, k, v, output gate)."""

    has_bias = False

    def __init__(self, cfg: DecayLinearAttentionConfig, width: int,
                 eps: float, dtype):
        super().__init__()
        self.cfg = cfg
        self.eps = eps
        self.dtype = dtype
        n, nv = cfg.heads * cfg.dim, cfg.heads * cfg.vdim
        self.in_sizes = [n, n, nv, nv]
        self.in_names = ["q", "k", "v", "g"]
        self.register_buffer(
            "decay", torch.tensor(cfg.decay, dtype=torch.float32),
            persistent=False)
        self.norm_w = _f32_param((nv,), 1.0)
        self.o_proj = RowParallelLinear(nv, width, dtype=dtype)

    def state_tensors(self, num_blocks, block_size, num_slots, device):
        c = self.cfg
        return {"lin": torch.zeros((num_slots, c.heads, c.dim, c.vdim),
                                   dtype=torch.float32, device=device)}

    def block_bytes(self, block_size: int) -> int:
        return 0

    def forward(self, parts, meta, cache) -> torch.Tensor:
        q, k, v, g = parts
        c = self.cfg
        o_raw = seqmix.decay_linear_attention(
            q, k, v, self.decay, cache["lin"], meta.seq_cu, meta.seq_slots,
            meta.positions, c.heads, c.dim, c.vdim, row_seq=meta.row_seq)
        o = seqmix.group_rms_gate(o_raw, g, self.norm_w, 1, self.eps,
                                  "sigmoid", self.dtype)
        return self.o_proj(o)


class TalkingWindowAttention(nn.Module):
    """Windowed softmax attention with head mixing; q/k/v biases ride the
    merged projection's bias."""

    has_bias = True

    def __init__(self, cfg: TalkingWindowAttentionConfig, width: int,
                 eps: float, dtype):
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        self.in_sizes = [cfg.heads * cfg.dim, cfg.kv_heads * cfg.dim,
                         cfg.kv_heads * cfg.vdim]
        self.in_names = ["q", "k", "v"]
        self.r1 = _f32_param((cfg.heads,), 0.0)
        self.r2 = _f32_param((cfg.heads,), 0.0)
        self.talk = nn.Parameter(torch.eye(cfg.heads, dtype=torch.float32),
                                 requires_grad=False)
        self.o_proj = RowParallelLinear(cfg.heads * cfg.vdim, width,
                                        dtype=dtype)
        self.o_bias = nn.Parameter(torch.zeros(width, dtype=dtype),
                                   requires_grad=False)

    def state_tensors(self, num_blocks, block_size, num_slots, device):
        c = self.cfg
        return {
            "k": torch.zeros((num_blocks, c.kv_heads, block_size, c.dim),
                             dtype=self.dtype, device=device),
            "v": torch.zeros((num_blocks, c.kv_heads, block_size, c.vdim),
                             dtype=self.dtype, device=device),
        }

    def block_bytes(self, block_size: int) -> int:
        c = self.cfg
        esize = torch.empty((), dtype=self.dtype).element_size()
        return c.kv_heads * block_size * (c.dim + c.vdim) * esize

    def forward(self, parts, meta, cache) -> torch.Tensor:
        q, k, v = parts
        c = self.cfg
        seqmix.paged_cache_write_(k, v, cache["k"], cache["v"],
                                  meta.slot_mapping)
        o = seqmix.talking_window_attention(
            q, cache["k"], cache["v"], meta.seq_bt, meta.row_seq,
            meta.positions, c.scale, c.window, self.r1, self.r2, self.talk,
            c.heads, seq_cu=meta.seq_cu, tiles=meta.seq_tiles)
        return F.linear(o.view(o.shape[0], c.heads * c.vdim),
                        self.o_proj.weight, self.o_bias)


class GatedDeltaMixer(nn.Module):
    """Gated-delta-rule mixer: q, k, v (convolved), write strength, decay
    input and output gate come from the merged projection."""

    has_bias = False

    def __init__(self, cfg: GatedDeltaConfig, width: int, eps: float, dtype):
        super().__init__()
        self.cfg = cfg
        self.eps = eps
        self.dtype = dtype
        nq, nv = cfg.kv_heads * cfg.dim, cfg.heads * cfg.vdim
        self.channels = 2 * nq + nv
        # q | k | v stay adjacent: the convolution reads them as one block
        self.in_sizes = [nq, nq, nv, cfg.heads, cfg.heads, nv]
        self.in_names = ["q", "k", "v", "b", "a", "g"]
        conv = torch.zeros(self.channels, cfg.conv, dtype=torch.float32)
        conv[:, -1] = 1.0
        self.conv_w = nn.Parameter(conv, requires_grad=False)
        self.a_log = _f32_param((cfg.heads,), 0.0)
        self.dt_bias = _f32_param((cfg.heads,), 0.0)
        self.norm_w = _f32_param((cfg.vdim,), 1.0)
        self.o_proj = RowParallelLinear(nv, width, dtype=dtype)

    def state_tensors(self, num_blocks, block_size, num_slots, device):
        c = self.cfg
        return {
            "conv": torch.zeros((num_slots, max(c.conv - 1, 1), self.channels),
                                dtype=torch.float32, device=device),
            "delta": torch.zeros((num_slots, c.heads, c.dim, c.vdim),
                                 dtype=torch.float32, device=device),
        }

    def block_bytes(self, block_size: int) -> int:
        return 0

    def forward(self, parts, meta, cache) -> torch.Tensor:
        q, k, v, b, a, g = parts
        c = self.cfg
        # q|k|v as one strided view of the projection output
        x = torch.as_strided(
            q, (q.shape[0], self.channels), (q.stride(0), 1),
            q.storage_offset())
        o_raw = seqmix.gated_delta_rule(
            x, self.conv_w, a, b, self.a_log, self.dt_bias, cache["conv"],
            cache["delta"], meta.seq_cu, meta.seq_slots, meta.positions,
            c.heads, c.kv_heads, c.dim, c.vdim, row_seq=meta.row_seq)
        o = seqmix.group_rms_gate(o_raw, g, self.norm_w, c.heads, self.eps,
                                  "silu", self.dtype)
        return self.o_proj(o)


class RoutedExperts(nn.Module):
    """Mixture of feed-forward experts: down(silu(gate x) * up x)
    (``act`` "silu_gate"), down(relu(up x)^2) (``act`` "relu_sq") or the
    clamped gated unit down(g' sigmoid(1.702 g') (u' + 1)), g' = min(gate
    x, limit), u' = clamp(up x, -limit, limit) (``act`` "clamped_glu").

    Router logits are an fp32 product (plus an optional bias); scores are sigmoid(z) or
    softmax(z); the ``top`` largest are chosen, optionally divided by their
    sum (+1e-20), and multiplied by ``scale``. With ``groups`` = (count,
    keep) the router is group-limited: sigmoid scores, the choice runs on
    score + a per-expert correction inside the ``keep`` best of ``count``
    groups of neighbouring experts, and the weights are the chosen scores
    as they are. On the GPU the experts run
    as two grouped GEMMs over block-aligned expert segments: the MFMA
    kernel on packed bf16 weights where the sizes fit its tiles, the
    plain grouped kernel otherwise (fp32, odd sizes)."""

    def __init__(self, width: int, ff: int, experts: int, top: int, dtype,
                 score: str = "sigmoid", renorm: bool = True,
                 scale: float = 1.0, act: str = "silu_gate",
                 router_bias: bool = False, limit: float = 0.0,
                 groups: Optional[Tuple[int, int]] = None):
        super().__init__()
        if score not in ("sigmoid", "softmax"):
            raise ValueError(f"unknown router score {score!r}")
        if act not in ("silu_gate", "relu_sq", "clamped_glu"):
            raise ValueError(f"unknown expert activation {act!r}")
        self.act = act
        self.gated = act != "relu_sq"
        self.limit = float(limit)
        self.groups = None
        if groups is not None:
            count, keep = int(groups[0]), int(groups[1])
            if (count < 1 or experts % count or not 1 <= keep <= count
                    or top > keep * (experts // count)):
                raise ValueError(
                    f"router groups {groups} do not fit {experts} experts "
                    f"with top {top}")
            self.groups = (count, keep)
        if not 1 <= top <= experts:
            raise ValueError("top must be in 1..experts")
        self.width, self.ff, self.experts, self.top = width, ff, experts, top
        self.score, self.renorm, self.scale = score, renorm, float(scale)
        self.dtype = dtype
        self.router = nn.Parameter(
            torch.empty(experts, width, dtype=torch.float32).normal_(0, 0.02),
            requires_grad=False)
        self.router_bias = (_f32_param((experts,), 0.0) if router_bias
                            else None)
        # group-limited routing: added to the scores for the choice only
        self.correction = (_f32_param((experts,), 0.0)
                           if self.groups is not None else None)
        # gated: gate rows then up rows; otherwise the up rows alone
        self.gate_up = nn.Parameter(
            torch.empty(experts, (2 if self.gated else 1) * ff, width,
                        dtype=dtype).normal_(0, 0.02),
            requires_grad=False)
        self.down = nn.Parameter(
            torch.empty(experts, width, ff, dtype=dtype).normal_(0, 0.02),
            requires_grad=False)
        self._packed = None

    # the MFMA grouped GEMM wants bf16, K % 32 == 0 and whole column tiles
    def _mfma_fits(self) -> bool:
        return (self.dtype == torch.bfloat16 and self.width % 128 == 0
                and self.ff % 64 == 0 and self.experts <= 128)

    def invalidate_packed(self):
        """The expert weights changed (checkpoint load, tests): repack on
        next use."""
        self._packed_stale = True

    def _packed_weights(self):
        if self._packed is None or getattr(self, "_packed_stale", False):
            from fusioninfer_amd import ops

            fresh = (
                ops.pack_moe_weights(
                    self.gate_up.data.transpose(1, 2).contiguous()),
                ops.pack_moe_weights(
                    self.down.data.transpose(1, 2).contiguous()))
            if self._packed is None:
                self._packed = fresh
            else:
                # in place: captured decode graphs keep reading these
                # tensors
                for old, new in zip(self._packed, fresh):
                    old.copy_(new)
            self._packed_stale = False
        return self._packed

    def route(self, x):
        from fusioninfer_amd import ops

        logits = F.linear(x.float(), self.router, self.router_bias)
        if self.groups is not None:
            return ops.moe_route_grouped(logits, self.correction, self.top,
                                         self.groups[0], self.groups[1])
        return ops.moe_route(logits, self.top, self.score, self.renorm,
                             self.scale)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        from fusioninfer_amd import ops

        T = x.shape[0]
        topv, topi = self.route(x)
        if not x.is_cuda:
            out = torch.zeros(T, self.width, dtype=torch.float32)
            for e in range(self.experts):
                rows, kk = (topi == e).nonzero(as_tuple=True)
                if rows.numel() == 0:
                    continue
                gu = F.linear(x[rows], self.gate_up[e]).float()
                if self.act == "clamped_glu":
                    act = seqmix.clamped_glu(gu, self.limit).to(x.dtype)
                elif self.gated:
                    act = (F.silu(gu[:, : self.ff])
                           * gu[:, self.ff:]).to(x.dtype)
                else:
                    act = torch.relu(gu).pow(2).to(x.dtype)
                y = F.linear(act, self.down[e]).float()
                out.index_add_(0, rows, y * topv[rows, kk].unsqueeze(1))
            return out.to(x.dtype)
        E = self.experts
        fast = self._mfma_fits()
        block_m = 16
        if fast and T * self.top >= 64 * E:
            block_m = 128
        sorted_ids, expert_ids, n_valid, pos, PM = ops.moe_align(
            topi, 0, E, block_m)
        act = torch.empty(PM, self.ff, dtype=x.dtype, device=x.device)
        y = torch.empty(PM, self.width, dtype=x.dtype, device=x.device)
        up_act = None if self.act == "silu_gate" else self.act
        if fast:
            gu_p, dn_p = self._packed_weights()
            ops.moe_gemm(act, x, gu_p, sorted_ids, expert_ids, n_valid,
                         block_m, gate_up=self.gated, up_act=up_act,
                         limit=self.limit)
            ops.moe_gemm(y, act, dn_p, sorted_ids, expert_ids, n_valid,
                         block_m, gate_up=False)
        else:
            ops.moe_gemm_plain(act, x, self.gate_up, sorted_ids, expert_ids,
                               n_valid, block_m, gate_up=self.gated,
                               up_act=up_act, limit=self.limit)
            ops.moe_gemm_plain(y, act, self.down, sorted_ids, expert_ids,
                               n_valid, block_m, gate_up=False)
        out = torch.empty(T, self.width, dtype=x.dtype, device=x.device)
        ops.moe_combine(out, y, pos, topv.reshape(-1).contiguous())
        return out


class GatedResidualLayer(nn.Module):
    """x <- x + gate1 * sum_m scale_m mixer_m(h),  h = layer_norm(x) w1
    x <- x + gate2 * ff(h2),                       h2 = layer_norm(x) w2
    with gate = sigmoid(W h + b) per coordinate and the residual stream x
    kept in fp32. All input branches of all mixers and the first gate's W
    are one merged projection of h. ``forward`` receives h (this layer's
    normed input) and returns the NEXT layer's normed input, so every
    residual update is fused with the norm that follows it."""

    def __init__(self, mixers: Sequence[Tuple[str, nn.Module, float]],
                 mlp: Optional[nn.Module], width: int, eps: float, dtype):
        super().__init__()
        if not 1 <= len(mixers) <= 2:
            raise ValueError("one or two mixers per layer")
        self.names = [m[0] for m in mixers]
        self.mixers = nn.ModuleList([m[1] for m in mixers])
        self.scales = [float(m[2]) for m in mixers]
        self.mlp = mlp
        self.eps = eps
        self.dtype = dtype
        self.width = width
        self.branches: List[Tuple[str, str]] = []
        self.sizes: List[int] = []
        for name, mod in zip(self.names, self.mixers):
            for br, size in zip(mod.in_names, mod.in_sizes):
                self.branches.append((name, br))
                self.sizes.append(size)
        self.branches.append(("", "rg1"))
        self.sizes.append(width)
        self.in_proj = MergedColumnParallelLinear(
            width, self.sizes, dtype=dtype,
            bias=any(m.has_bias for m in self.mixers))
        self.norm1 = _f32_param((width,), 1.0)
        self.rg1_bias = _f32_param((width,), 0.0)
        if mlp is not None:
            self.norm2 = _f32_param((width,), 1.0)
            self.rg2 = ReplicatedLinear(width, width, dtype=dtype)
            self.rg2_bias = _f32_param((width,), 0.0)

    def in_proj_rows(self, mixer: str, branch: str):
        off = 0
        for key, size in zip(self.branches, self.sizes):
            if key == (mixer, branch):
                return off, size
            off += size
        raise KeyError((mixer, branch))

    def forward(self, resid, h, meta, cache, next_norm_w):
        parts = self.in_proj(h).split(self.sizes, dim=-1)
        ys, at = [], 0
        for mod in self.mixers:
            n = len(mod.in_sizes)
            ys.append(mod(parts[at: at + n], meta, cache))
            at += n
        w_after = self.norm2 if self.mlp is not None else next_norm_w
        h2 = seqmix.gated_residual_layer_norm_(
            resid, ys[0], self.scales[0],
            ys[1] if len(ys) > 1 else None,
            self.scales[1] if len(ys) > 1 else 0.0,
            parts[-1], self.rg1_bias, w_after, self.eps, self.dtype)
        if self.mlp is None:
            return h2
        return seqmix.gated_residual_layer_norm_(
            resid, self.mlp(h2), 1.0, None, 0.0, self.rg2(h2), self.rg2_bias,
            next_norm_w, self.eps, self.dtype)


# ------------------------------------------------------------------------
# Parallel-residual family of blocks


@dataclasses.dataclass
class TemperedGatedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                 # per-head query/key size
    vdim: int                # per-head value size
    scale: float             # score multiplier
    temp_coef: float = 0.0   # query factor 1 + coef * ln(floor((p+1)/every)+1)
    temp_every: int = 0      # 0: no query temperature

    def __post_init__(self):
        if self.heads % self.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")


@dataclasses.dataclass
class LatentAttentionConfig:
    heads: int
    dim: int                 # unrotated query/key size per head
    rot_dim: int             # rotated query/key size (key part shared)
    vdim: int
    rank: int                # size of the cached latent
    scale: float
    rot_base: float
    sink: bool = True        # learned per-head term in the denominator
    rot_dims: int = -1       # leading entries of the rotated part that turn
                             # (-1: all of it)

    def __post_init__(self):
        if self.rot_dims < 0:
            self.rot_dims = self.rot_dim
        if self.rot_dim % 2 or self.rot_dims % 2:
            raise ValueError("rot_dim and rot.dims must be even")
        if self.rot_dims > self.rot_dim:
            raise ValueError("rot.dims exceeds rot_dim")


@dataclasses.dataclass
class RGLRUConfig:
    width: int               # channels of the recurrence
    blocks: int              # block-diagonal gate matrices
    conv: int                # taps of the causal convolution
    # log a = -decay_scale * r * softplus(lam): the unit's fixed constant
    decay_scale: float = 8.0

    def __post_init__(self):
        if self.width % self.blocks:
            raise ValueError("width must be a multiple of blocks")
        if self.conv < 1:
            raise ValueError("conv taps must be >= 1")


class TemperedGatedAttention(nn.Module):
    """q, k, v and the per-head gate come from the merged projection (the
    gate's rows carry a zero bias)."""

    has_bias = True
    biased = ("q", "k", "v")

    def __init__(self, cfg: TemperedGatedAttentionConfig, width: int,
                 eps: float, dtype):
        super().__init__()
        self.cfg = cfg
        self.eps = eps
        self.dtype = dtype
        self.in_sizes = [cfg.heads * cfg.dim, cfg.kv_heads * cfg.dim,
                         cfg.kv_heads * cfg.vdim, cfg.heads]
        self.in_names = ["q", "k", "v", "g"]
        self.q_norm = _f32_param((cfg.dim,), 1.0)
        self.k_norm = _f32_param((cfg.dim,), 1.0)
        self.o_proj = RowParallelLinear(cfg.heads * cfg.vdim, width,
                                        dtype=dtype)

    def state_tensors(self, num_blocks, block_size, num_slots, device):
        c = self.cfg
        return {
            "k": torch.zeros((num_blocks, c.kv_heads, block_size, c.dim),
                             dtype=self.dtype, device=device),
            "v": torch.zeros((num_blocks, c.kv_heads, block_size, c.vdim),
                             dtype=self.dtype, device=device),
        }

    def block_bytes(self, block_size: int) -> int:
        c = self.cfg
        esize = torch.empty((), dtype=self.dtype).element_size()
        return c.kv_heads * block_size * (c.dim + c.vdim) * esize

    def forward(self, parts, meta, cache) -> torch.Tensor:
        q, k, v, g = parts
        c = self.cfg
        qn = seqmix.headnorm_qtemp_cache_(
            q, k, v, meta.positions, self.q_norm, self.k_norm, self.eps,
            c.temp_coef, c.temp_every, cache["k"], cache["v"],
            meta.slot_mapping, c.heads, c.kv_heads, c.dim, c.vdim)
        o = seqmix.sink_paged_attention(
            qn, cache["k"], cache["v"], meta.seq_bt, meta.row_seq,
            meta.positions, c.scale, out_gate=g, seq_cu=meta.seq_cu,
            tiles=meta.seq_tiles)
        return self.o_proj(o.view(o.shape[0], c.heads * c.vdim))


class LatentAttention(nn.Module):
    """q and the down projection (latent | shared rotated key part) come
    from the merged projection. The key expansion is folded into the
    queries (q_h^T W_uk,h) and the value expansion applied to the attended
    latents, so attention runs over the cached rows [latent | rotated
    part] with one shared key/value head."""

    has_bias = False

    def __init__(self, cfg: LatentAttentionConfig, width: int, eps: float,
                 dtype):
        super().__init__()
        self.cfg = cfg
        self.eps = eps
        self.dtype = dtype
        H = cfg.heads
        self.in_sizes = [H * (cfg.dim + cfg.rot_dim), cfg.rank + cfg.rot_dim]
        self.in_names = ["q", "dkv"]
        self.c_norm = _f32_param((cfg.rank,), 1.0)
        self.uk = nn.Parameter(
            torch.empty(H * cfg.dim, cfg.rank, dtype=dtype).normal_(0, 0.02),
            requires_grad=False)
        self.uv = nn.Parameter(
            torch.empty(H * cfg.vdim, cfg.rank, dtype=dtype).normal_(0, 0.02),
            requires_grad=False)
        self.sink = _f32_param((H,), 0.0) if cfg.sink else None
        self.o_proj = RowParallelLinear(H * cfg.vdim, width, dtype=dtype)
        self.register_buffer(
            "inv_freq", rotary_inv_freq(cfg.rot_dims, cfg.rot_base),
            persistent=False)

    def state_tensors(self, num_blocks, block_size, num_slots, device):
        c = self.cfg
        return {"kv": torch.zeros(
            (num_blocks, 1, block_size, c.rank + c.rot_dim),
            dtype=self.dtype, device=device)}

    def block_bytes(self, block_size: int) -> int:
        c = self.cfg
        esize = torch.empty((), dtype=self.dtype).element_size()
        return block_size * (c.rank + c.rot_dim) * esize

    def forward(self, parts, meta, cache) -> torch.Tensor:
        q, dkv = parts
        c = self.cfg
        T, H = q.shape[0], c.heads
        qf = torch.empty((T, H, c.rank + c.rot_dim), dtype=q.dtype,
                         device=q.device)
        seqmix.latent_rope_cache_(
            q, dkv, meta.positions, self.inv_freq, self.c_norm, self.eps,
            cache["kv"], meta.slot_mapping, H, c.dim, c.rot_dim, c.rank, qf)
        # fold the key expansion into the queries: [H, T, dim] x [H, dim, rank]
        qu = q.view(T, H, c.dim + c.rot_dim)[:, :, : c.dim].transpose(0, 1)
        torch.bmm(qu, self.uk.view(H, c.dim, c.rank),
                  out=qf.transpose(0, 1)[:, :, : c.rank])
        o = seqmix.sink_paged_attention(
            qf, cache["kv"], None, meta.seq_bt, meta.row_seq, meta.positions,
            c.scale, sink=self.sink, value_dims=c.rank, seq_cu=meta.seq_cu,
            tiles=meta.seq_tiles)
        # expand the attended latents: [H, T, rank] x [H, rank, vdim]
        ov = torch.empty((T, H, c.vdim), dtype=q.dtype, device=q.device)
        torch.bmm(o.transpose(0, 1),
                  self.uv.view(H, c.vdim, c.rank).transpose(1, 2),
                  out=ov.transpose(0, 1))
        return self.o_proj(ov.view(T, H * c.vdim))


class RGLRUMixer(nn.Module):
    """Recurrent block: the GELU branch and the convolved branch come from
    the merged projection (both with biases). The block-diagonal gate
    products run in fp32 as one batched GEMM."""

    has_bias = True
    biased = ("y", "x")

    def __init__(self, cfg: RGLRUConfig, width: int, eps: float, dtype):
        super().__init__()
        self.cfg = cfg
        self.dtype = dtype
        W, B = cfg.width, cfg.blocks
        bw = W // B
        self.in_sizes = [W, W]
        self.in_names = ["y", "x"]
        conv = torch.zeros(W, cfg.conv, dtype=torch.float32)
        conv[:, -1] = 1.0
        self.conv_w = nn.Parameter(conv, requires_grad=False)
        self.conv_b = _f32_param((W,), 0.0)
        # per block: recurrence-gate rows then input-gate rows, [out, in]
        self.gate_w = nn.Parameter(
            torch.empty(B, 2 * bw, bw, dtype=torch.float32).normal_(
                0, 1.0 / math.sqrt(bw)), requires_grad=False)
        self.gate_b = _f32_param((B, 2 * bw), 0.0)
        self.lam = _f32_param((W,), 0.0)
        self.o_proj = RowParallelLinear(W, width, dtype=dtype)

    def state_tensors(self, num_blocks, block_size, num_slots, device):
        c = self.cfg
        return {
            "conv": torch.zeros((num_slots, max(c.conv - 1, 1), c.width),
                                dtype=torch.float32, device=device),
            "lru": torch.zeros((num_slots, c.width), dtype=torch.float32,
                               device=device),
        }

    def block_bytes(self, block_size: int) -> int:
        return 0

    def forward(self, parts, meta, cache) -> torch.Tensor:
        y_lin, x_lin = parts
        c = self.cfg
        T, B = y_lin.shape[0], c.blocks
        u = seqmix.causal_conv_state(
            x_lin, self.conv_w, self.conv_b, cache["conv"], meta.seq_cu,
            meta.row_seq, meta.seq_slots, meta.positions)
        gates = torch.bmm(u.view(T, B, c.width // B).transpose(0, 1),
                          self.gate_w.transpose(1, 2))
        o = seqmix.rglru_scan(
            u, gates, self.gate_b, self.lam, y_lin, cache["lru"],
            meta.seq_cu, meta.seq_slots, meta.positions, c.decay_scale,
            self.dtype, max_rows=meta.max_seq_rows)
        return self.o_proj(o)


class SquaredReluMLP(nn.Module):
    """down(relu(up x)^2). With ``own_up`` False the up projection is a
    branch of the caller's merged projection and forward takes its
    result."""

    def __init__(self, width: int, ff: int, dtype, own_up: bool = True):
        super().__init__()
        self.ff = ff
        self.up_proj = (ReplicatedLinear(width, ff, dtype=dtype)
                        if own_up else None)
        self.down_proj = RowParallelLinear(ff, width, dtype=dtype)

    def forward(self, x):
        if self.up_proj is not None:
            x = self.up_proj(x)
        return self.down_proj(seqmix.relu_squared(x))


class ParallelResidualLayer(nn.Module):
    """x <- x + mult * (mixer(h) + ff(h)),  h = layer_norm(x) w,
    with the residual stream x kept in fp32. The mixer's input branches
    and the up projection of the dense feed-forward (or of the shared
    expert) are one merged projection of h; routed experts read h
    themselves. ``forward`` receives h and returns the next layer's normed
    input (None when ``next_norm_w`` is None), so the residual update is
    fused with the norm that follows it."""

    def __init__(self, mixer: nn.Module, dense: Optional[SquaredReluMLP],
                 routed: Optional[nn.Module], width: int, eps: float,
                 mult: float, dtype):
        super().__init__()
        self.mixer = mixer
        self.dense = dense          # dense feed-forward or shared expert
        self.routed = routed
        self.eps = eps
        self.mult = float(mult)
        self.dtype = dtype
        self.width = width
        self.branches: List[str] = list(mixer.in_names)
        self.sizes: List[int] = list(mixer.in_sizes)
        if dense is not None:
            self.branches.append("up")
            self.sizes.append(dense.ff)
        self.in_proj = MergedColumnParallelLinear(
            width, self.sizes, dtype=dtype, bias=mixer.has_bias)
        self.norm1 = _f32_param((width,), 1.0)

    def in_proj_rows(self, branch: str):
        off = 0
        for name, size in zip(self.branches, self.sizes):
            if name == branch:
                return off, size
            off += size
        raise KeyError(branch)

    def forward(self, resid, h, meta, cache, next_norm_w):
        parts = self.in_proj(h).split(self.sizes, dim=-1)
        n = len(self.mixer.in_sizes)
        ys = [self.mixer(parts[:n], meta, cache)]
        if self.dense is not None:
            ys.append(self.dense(parts[n]))
        if self.routed is not None:
            ys.append(self.routed(h))
        return seqmix.scaled_residual_layer_norm_(
            resid, ys, [self.mult] * len(ys), next_norm_w, self.eps,
            self.dtype)


# ------------------------------------------------------------------------
# Post-norm family of blocks


@dataclasses.dataclass
class WindowedSinkAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                 # per-head query/key size
    vdim: int                # per-head value size
    scale: float             # score multiplier
    window: int = 0          # 0: plain causal; else p - j < window ...
    keep_first: int = 0      # ... or j < keep_first
    rot_dims: int = 0        # leading entries of a head that turn (0: none)
    rot_base: float = 10000.0
    # frequency blend for context extension (rot_original 0: none)
    rot_factor: float = 1.0
    rot_original: float = 0.0
    rot_fast: float = 0.0
    rot_slow: float = 0.0

    def __post_init__(self):
        if self.heads % self.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if self.rot_dims % 2 or self.rot_dims > self.dim:
            raise ValueError("rot.dims must be even and at most dim")
        if self.window < 0 or self.keep_first < 0:
            raise ValueError("window and keep_first must not be negative")


class WindowedSinkAttention(nn.Module):
    """q, k, v and the elementwise gate come from the caller's merged
    projection (the gate's rows carry a zero bias). With ``own_kv`` False
    the block has neither key nor value branches and ``forward`` is handed
    the cache of the layer it borrows from."""

    has_bias = True
    biased = ("q", "k", "v")

    def __init__(self, cfg: WindowedSinkAttentionConfig, width: int,
                 eps: float, dtype, own_kv: bool = True):
        super().__init__()
        self.cfg = cfg
        self.eps = eps
        self.dtype = dtype
        self.own_kv = own_kv
        H, G = cfg.heads, cfg.kv_heads
        if own_kv:
            self.in_names = ["q", "k", "v", "g"]
            self.in_sizes = [H * cfg.dim, G * cfg.dim, G * cfg.vdim,
                             H * cfg.vdim]
        else:
            self.in_names = ["q", "g"]
            self.in_sizes = [H * cfg.dim, H * cfg.vdim]
        self.q_norm = _f32_param((H * cfg.dim,), 1.0)
        self.k_norm = _f32_param((G * cfg.dim,), 1.0) if own_kv else None
        self.sink = _f32_param((H,), 0.0)
        self.o_proj = RowParallelLinear(H * cfg.vdim, width, dtype=dtype)
        if cfg.rot_dims:
            inv_freq, mult = seqmix.blended_rotary(
                cfg.rot_dims, cfg.rot_base, cfg.rot_factor, cfg.rot_original,
                cfg.rot_fast, cfg.rot_slow)
        else:
            inv_freq, mult = torch.zeros(0, dtype=torch.float32), 1.0
        self.rot_mult = float(mult)
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    def state_tensors(self, num_blocks, block_size, num_slots, device):
        if not self.own_kv:
            return {}
        c = self.cfg
        return {
            "k": torch.zeros((num_blocks, c.kv_heads, block_size, c.dim),
                             dtype=self.dtype, device=device),
            "v": torch.zeros((num_blocks, c.kv_heads, block_size, c.vdim),
                             dtype=self.dtype, device=device),
        }

    def block_bytes(self, block_size: int) -> int:
        if not self.own_kv:
            return 0
        c = self.cfg
        esize = torch.empty((), dtype=self.dtype).element_size()
        return c.kv_heads * block_size * (c.dim + c.vdim) * esize

    def forward(self, parts, meta, cache) -> torch.Tensor:
        c = self.cfg
        if self.own_kv:
            q, k, v, g = parts
        else:
            (q, g), k, v = parts, None, None
        qn = seqmix.widenorm_rope_cache_(
            q, k, v, meta.positions, self.q_norm, self.k_norm, self.eps,
            self.inv_freq, self.rot_mult, cache["k"], cache["v"],
            meta.slot_mapping, c.heads, c.kv_heads, c.dim, c.vdim)
        o = seqmix.sink_paged_attention(
            qn, cache["k"], cache["v"], meta.seq_bt, meta.row_seq,
            meta.positions, c.scale, sink=self.sink, out_gate=g,
            seq_cu=meta.seq_cu, tiles=meta.seq_tiles, window=c.window,
            keep_first=c.keep_first)
        return self.o_proj(o.view(o.shape[0], c.heads * c.vdim))


class ClampedGatedMLP(nn.Module):
    """down(g' sigmoid(1.702 g') (u' + 1)), g' = min(gate x, limit),
    u' = clamp(up x, -limit, limit); gate and up are one merged GEMM."""

    def __init__(self, width: int, ff: int, limit: float, dtype):
        super().__init__()
        self.ff = ff
        self.limit = float(limit)
        self.gate_up_proj = MergedColumnParallelLinear(width, [ff, ff],
                                                       dtype=dtype)
        self.down_proj = RowParallelLinear(ff, width, dtype=dtype)

    def forward(self, x):
        return self.down_proj(
            seqmix.clamped_glu(self.gate_up_proj(x), self.limit))


class PostNormLayer(nn.Module):
    """x <- x + LN1(mixer(x)); x <- x + LN2(ff(x)) on an fp32 stream x.
    The sublayers read x itself (rounded to the activation dtype); the
    layer norms carry weight and bias and sit on the sublayer outputs, so
    each is one kernel with the residual sum. ``forward`` receives and
    returns the activation-dtype copy of the stream."""

    def __init__(self, mixer: nn.Module, mlp: Optional[nn.Module],
                 width: int, eps: float, dtype):
        super().__init__()
        self.mixer = mixer
        self.mlp = mlp
        self.eps = eps
        self.dtype = dtype
        self.branches: List[str] = list(mixer.in_names)
        self.sizes: List[int] = list(mixer.in_sizes)
        self.in_proj = MergedColumnParallelLinear(
            width, self.sizes, dtype=dtype, bias=mixer.has_bias)
        self.norm1 = _f32_param((width,), 1.0)
        self.norm1_b = _f32_param((width,), 0.0)
        if mlp is not None:
            self.norm2 = _f32_param((width,), 1.0)
            self.norm2_b = _f32_param((width,), 0.0)

    def in_proj_rows(self, branch: str):
        off = 0
        for name, size in zip(self.branches, self.sizes):
            if name == branch:
                return off, size
            off += size
        raise KeyError(branch)

    def forward(self, resid, x, meta, cache):
        parts = self.in_proj(x).split(self.sizes, dim=-1)
        y = self.mixer(parts, meta, cache)
        x = seqmix.post_norm_residual_(resid, y, self.norm1, self.norm1_b,
                                       self.eps, self.dtype)
        if self.mlp is None:
            return x
        return seqmix.post_norm_residual_(resid, self.mlp(x), self.norm2,
                                          self.norm2_b, self.eps, self.dtype)

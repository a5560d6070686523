"""Kazozen: a decoder-only design of post-norm attention layers.

The stream starts as ``embed[token] * c`` plus a row of a hashed
(previous token, token) table. Every layer adds the layer-normed OUTPUT of
its sublayers, ``x += LN1(mixer(x))``, ``x += LN2(ff(x))``; the sublayers
read x itself. The mixer is grouped-query attention with projection
biases, one RMS norm over the whole query / key projection, interleaved
partial rotary positions with blended frequencies, a sliding window that
keeps the first keys, a per-head softmax sink and an elementwise sigmoid
gate; a layer may read the paged keys and values of an earlier layer
instead of projecting its own. The feed-forward is a clamped gated unit,
dense or as group-limited routed experts, or absent. The head is the
embedding table itself; logits pass through ``cap * tanh(z / cap)``.

This module only ASSEMBLES the design from the reusable blocks in
``models/mixers.py``: it parses ``config.json``, declares what cache and
state every layer needs (paged k/v for layers that project their own, the
previous token per state slot), and maps checkpoint tensor names onto the
merged parameters. The engine's block manager, state-slot manager,
scheduler and sampler serve it like any other model.
"""

from __future__ import annotations

import dataclasses
from typing import Dict, Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from fusioninfer_amd.config import ModelConfig
from fusioninfer_amd.distributed import parallel_state as ps
from fusioninfer_amd.models.mixers import (
    ClampedGatedMLP,
    PostNormLayer,
    RoutedExperts,
    WindowedSinkAttention,
    WindowedSinkAttentionConfig,
)
from fusioninfer_amd.ops import seqmix

ARCHITECTURE = "Kazozen"


@dataclasses.dataclass
class FeedForwardConfig:
    kind: str                       # dense | moe
    ff: int                         # dense: hidden size; moe: per expert
    limit: float
    experts: int = 0
    top: int = 0
    groups: Optional[Tuple[int, int]] = None   # (count, keep)


@dataclasses.dataclass
class KazozenLayerConfig:
    mixer: WindowedSinkAttentionConfig
    kv_from: Optional[int]          # layer whose keys/values this one reads
    mlp: Optional[FeedForwardConfig]


@dataclasses.dataclass
class PairEmbeddingConfig:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclasses.dataclass
class KazozenConfig:
    width: int
    vocab: int
    eps: float
    embed_scale: float
    pair: Optional[PairEmbeddingConfig]
    logit_cap: float                # 0: logits are not capped
    layers: List[KazozenLayerConfig]


def _parse_mlp(i: int, mlp: Optional[dict]) -> Optional[FeedForwardConfig]:
    if not mlp:
        return None
    kind = mlp.get("kind")
    if kind == "dense":
        return FeedForwardConfig("dense", int(mlp["ff"]), float(mlp["limit"]))
    if kind == "moe":
        r, e = mlp["router"], mlp["expert"]
        g = r.get("groups")
        return FeedForwardConfig(
            "moe", int(e["ff"]), float(e["limit"]), experts=int(r["experts"]),
            top=int(r["top"]),
            groups=(int(g["count"]), int(g["keep"])) if g else (1, 1))
    raise ValueError(f"layer {i}: unknown mlp kind {kind!r}")


def _parse_mixer(m: dict) -> WindowedSinkAttentionConfig:
    mask = m.get("mask") or {}
    rot = m.get("rot") or {}
    sc = rot.get("scaling") or {}
    return WindowedSinkAttentionConfig(
        heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
        dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
        scale=float(m["scale"]),
        window=int(mask.get("size", 0)),
        keep_first=int(mask.get("keep_first", 0)),
        rot_dims=int(rot.get("dims", 0)) if rot else 0,
        rot_base=float(rot.get("base", 10000.0)),
        rot_factor=float(sc.get("factor", 1.0)),
        rot_original=float(sc.get("original", 0.0)),
        rot_fast=float(sc.get("fast", 0.0)),
        rot_slow=float(sc.get("slow", 0.0)))


def parse_config(raw: dict) -> KazozenConfig:
    """config.json -> KazozenConfig; every size and constant is read from
    the config."""
    layers = []
    for i, L in enumerate(raw["layers"]):
        if L.get("type") != "attention":
            raise ValueError(f"layer {i}: unknown mixer type {L.get('type')!r}")
        m = L["mixer"]
        mixer = _parse_mixer(m)
        src = m.get("kv_from")
        if src is not None:
            src = int(src)
            if not 0 <= src < i or layers[src].kv_from is not None:
                raise ValueError(
                    f"layer {i}: kv_from {src} must name an earlier layer "
                    "with keys and values of its own")
            o = layers[src].mixer
            if (o.kv_heads, o.dim, o.vdim) != (mixer.kv_heads, mixer.dim,
                                               mixer.vdim):
                raise ValueError(
                    f"layer {i}: key/value sizes differ from layer {src}'s")
        layers.append(KazozenLayerConfig(mixer, src,
                                         _parse_mlp(i, L.get("mlp"))))
    emb = raw.get("embedding") or {}
    bg = emb.get("bigram")
    return KazozenConfig(
        width=int(raw["width"]), vocab=int(raw["vocab"]),
        eps=float(raw["norm"]["eps"]),
        embed_scale=float(emb.get("scale", 1.0)),
        pair=PairEmbeddingConfig(int(bg["buckets"]), int(bg["mul_prev"]),
                                 int(bg["mul_cur"])) if bg else None,
        logit_cap=float(raw.get("logit_softcap") or 0.0),
        layers=layers)


def model_config_from_dict(raw: dict, model_path: Optional[str] = None,
                           name: str = ARCHITECTURE) -> ModelConfig:
    """Engine-level ModelConfig for a Kazozen config dict (the registry's
    architecture hook)."""
    arch = parse_config(raw)
    first = arch.layers[0].mixer
    ffs = [L.mlp for L in arch.layers if L.mlp is not None]
    return ModelConfig(
        name=name,
        architecture=ARCHITECTURE,
        arch=arch,
        hidden_size=arch.width,
        num_layers=len(arch.layers),
        num_heads=first.heads,
        num_kv_heads=first.kv_heads,
        head_dim=first.dim,
        intermediate_size=max((f.ff for f in ffs), default=0),
        vocab_size=arch.vocab,
        rms_norm_eps=arch.eps,
        qk_norm=False,
        model_path=model_path,
        max_position_embeddings=1 << 24,
    )


class KazozenLM(nn.Module):
    """pair embedding -> post-norm layers -> final layer norm -> tied head
    with capped logits.

    Engine interface (same as CausalLM): ``forward(ids, meta, caches)``
    returns the final-normed hidden rows, ``compute_logits`` applies the
    head. ``allocate_caches`` hands out one dict per layer (a borrowing
    layer gets the dict of the layer it reads); the previous token of
    every live sequence sits in a slot-indexed int32 tensor, so
    ``uses_state_slots`` makes the scheduler hand out state slots and the
    runner build sequence-grouped metadata."""

    uses_state_slots = True
    supports_prefix_caching = False   # the previous token has no block form

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        assert ps.tp_world_size() == 1 and ps.pp_world_size() == 1, (
            "Kazozen runs single-rank (TP/PP sharding of its mixers is "
            "not implemented)")
        self.cfg = cfg
        arch: KazozenConfig = cfg.arch
        self.arch = arch
        dtype = {"bfloat16": torch.bfloat16,
                 "float32": torch.float32}[cfg.dtype]
        self.dtype = dtype
        self.pp_first = self.pp_last = True
        W = arch.width
        base_seed = torch.initial_seed() % (2**62)
        torch.manual_seed(base_seed + 1000003)
        self.embed_tokens = nn.Parameter(
            torch.empty(arch.vocab, W, dtype=dtype).normal_(0.0, 0.02),
            requires_grad=False)
        self.pair_table = None
        if arch.pair is not None:
            self.pair_table = nn.Parameter(
                torch.empty(arch.pair.buckets + 1, W,
                            dtype=dtype).normal_(0.0, 0.02),
                requires_grad=False)
        layers = []
        for i, L in enumerate(arch.layers):
            torch.manual_seed(base_seed + 1000003 * (i + 2))
            mixer = WindowedSinkAttention(L.mixer, W, arch.eps, dtype,
                                          own_kv=L.kv_from is None)
            mlp = None
            if L.mlp is not None and L.mlp.kind == "dense":
                mlp = ClampedGatedMLP(W, L.mlp.ff, L.mlp.limit, dtype)
            elif L.mlp is not None:
                mlp = RoutedExperts(
                    W, L.mlp.ff, L.mlp.experts, L.mlp.top, dtype,
                    score="sigmoid", renorm=False, act="clamped_glu",
                    limit=L.mlp.limit, groups=L.mlp.groups)
            layers.append(PostNormLayer(mixer, mlp, W, arch.eps, dtype))
        self.layers = nn.ModuleList(layers)
        self.final_norm = nn.Parameter(torch.ones(W, dtype=torch.float32),
                                       requires_grad=False)
        self.final_norm_b = nn.Parameter(torch.zeros(W, dtype=torch.float32),
                                         requires_grad=False)
        torch.manual_seed(base_seed + 777)
        # when set to a list, forward appends the residual stream after
        # every layer (debugging, layer-by-layer tests)
        self.residual_trace: Optional[list] = None

    # ------------------------------------------------------ engine hooks
    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def kv_block_bytes(self, block_size: int) -> int:
        return max(sum(layer.mixer.block_bytes(block_size)
                       for layer in self.layers), 1)

    def allocate_caches(self, num_blocks: int, block_size: int,
                        num_slots: int, device) -> list:
        """One dict per layer: paged k/v of its attention, or the dict of
        the layer it borrows from. The first dict also holds the previous
        token of every state slot."""
        caches: list = []
        for layer, L in zip(self.layers, self.arch.layers):
            if L.kv_from is not None:
                caches.append(caches[L.kv_from])
            else:
                caches.append(layer.mixer.state_tensors(
                    num_blocks, block_size, num_slots, device))
        caches[0]["prev_token"] = torch.zeros(
            max(num_slots, 1), dtype=torch.int32, device=device)
        return caches

    # ----------------------------------------------------------- forward
    def forward(self, input_ids, meta, caches, hidden=None, residual=None):
        a = self.arch
        p = a.pair
        resid, x = seqmix.pair_embed(
            input_ids, self.embed_tokens, a.embed_scale, self.pair_table,
            p.buckets if p else 1, p.mul_prev if p else 0,
            p.mul_cur if p else 0, caches[0]["prev_token"], meta.seq_cu,
            meta.row_seq, meta.seq_slots, meta.positions, self.dtype)
        for layer, cache in zip(self.layers, caches):
            x = layer(resid, x, meta, cache)
            if self.residual_trace is not None:
                self.residual_trace.append(resid.detach().clone())
        return seqmix.layer_norm_affine(resid, self.final_norm,
                                        self.final_norm_b, a.eps, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = F.linear(hidden, self.embed_tokens).float()
        if self.arch.logit_cap > 0:
            seqmix.tanh_cap_(logits, self.arch.logit_cap)
        return logits

    # ----------------------------------------------------------- weights
    def load_weights(self, tensors: Iterable[Tuple[str, torch.Tensor]]) -> int:
        """Checkpoint names -> parameters. A layer's q/k/v/gate matrices
        land in its merged projection, expert matrices in the stacked
        expert tensors, gate and up of a dense unit in one merged matrix;
        norm weights and biases, sinks and the router correction are kept
        in fp32."""
        n = 0
        seen = set()
        for name, t in tensors:
            self._load_one(name, t)
            seen.add(name)
            n += 1
        missing = [k for k in self.expected_tensor_names() if k not in seen]
        if missing:
            raise ValueError(f"checkpoint lacks tensors: {missing[:8]}"
                             f"{' ...' if len(missing) > 8 else ''}")
        for layer in self.layers:
            if isinstance(layer.mlp, RoutedExperts):
                layer.mlp.invalidate_packed()
        return n

    def expected_tensor_names(self) -> List[str]:
        return list(self._name_map())

    def _name_map(self) -> Dict[str, tuple]:
        """checkpoint name -> (parameter, view spec or None)."""
        out: Dict[str, tuple] = {
            "embed": (self.embed_tokens, None),
            "final.norm": (self.final_norm, None),
            "final.norm.b": (self.final_norm_b, None),
        }
        if self.pair_table is not None:
            out["bigram"] = (self.pair_table, None)
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            mp = p + "mix."
            mod = layer.mixer
            out[p + "norm1"] = (layer.norm1, None)
            out[p + "norm1.b"] = (layer.norm1_b, None)
            for br in mod.in_names:
                rows = layer.in_proj_rows(br)
                out[mp + br] = (layer.in_proj.weight, rows)
                if br in mod.biased:
                    out[mp + br + ".b"] = (layer.in_proj.bias, rows)
            out[mp + "q.norm"] = (mod.q_norm, None)
            if mod.own_kv:
                out[mp + "k.norm"] = (mod.k_norm, None)
            out[mp + "sink"] = (mod.sink, None)
            out[mp + "o"] = (mod.o_proj.weight, None)
            fp = p + "mlp."
            mlp = layer.mlp
            if mlp is None:
                continue
            out[p + "norm2"] = (layer.norm2, None)
            out[p + "norm2.b"] = (layer.norm2_b, None)
            if isinstance(mlp, RoutedExperts):
                out[fp + "router"] = (mlp.router, None)
                out[fp + "correction"] = (mlp.correction, None)
                for e in range(mlp.experts):
                    out[f"{fp}e{e}.gate"] = (mlp.gate_up,
                                             ("idx", e, 0, mlp.ff))
                    out[f"{fp}e{e}.up"] = (mlp.gate_up,
                                           ("idx", e, mlp.ff, mlp.ff))
                    out[f"{fp}e{e}.down"] = (mlp.down, ("idx", e))
            else:
                out[fp + "gate"] = (mlp.gate_up_proj.weight, (0, mlp.ff))
                out[fp + "up"] = (mlp.gate_up_proj.weight, (mlp.ff, mlp.ff))
                out[fp + "down"] = (mlp.down_proj.weight, None)
        return out

    @staticmethod
    def _view(param, spec):
        dst = param.data
        if spec is None:
            return dst
        if spec[0] == "idx":
            dst = dst[spec[1]]
            return dst if len(spec) == 2 else dst[spec[2]: spec[2] + spec[3]]
        return dst[spec[0]: spec[0] + spec[1]]

    def _load_one(self, name: str, t: torch.Tensor) -> None:
        names = getattr(self, "_names", None)
        if names is None:
            names = self._names = self._name_map()
        if name not in names:
            raise ValueError(f"unknown tensor {name!r}")
        param, spec = names[name]
        dst = self._view(param, spec)
        if dst.shape != t.shape:
            raise ValueError(f"{name}: shape {tuple(t.shape)} does not fit "
                             f"{tuple(dst.shape)}")
        dst.copy_(t.to(dst.dtype))

    def export_weights(self) -> Dict[str, torch.Tensor]:
        """Inverse of load_weights (checkpoint naming), for writing
        random-init models to disk."""
        return {k: self._view(p, spec).detach().clone().contiguous()
                for k, (p, spec) in self._name_map().items()}

    def randomize_small_params(self, seed: int = 0) -> None:
        """Random-init use (benchmarks, tests): give norm weights, biases,
        sinks and corrections non-trivial values so every branch
        contributes."""
        g = torch.Generator().manual_seed(seed)

        def rnd(p, lo, hi):
            p.data.copy_((torch.rand(p.shape, generator=g) * (hi - lo) + lo)
                         .to(device=p.device, dtype=p.dtype))

        rnd(self.final_norm, 0.8, 1.2)
        rnd(self.final_norm_b, -0.1, 0.1)
        for layer in self.layers:
            mod = layer.mixer
            rnd(layer.norm1, 0.5, 1.5)
            rnd(layer.norm1_b, -0.1, 0.1)
            rnd(layer.in_proj.bias, -0.1, 0.1)
            a, n = layer.in_proj_rows("g")
            layer.in_proj.bias.data[a: a + n] = 0
            rnd(mod.q_norm, 0.5, 1.5)
            if mod.own_kv:
                rnd(mod.k_norm, 0.5, 1.5)
            rnd(mod.sink, -1.0, 2.0)
            if layer.mlp is not None:
                rnd(layer.norm2, 0.5, 1.5)
                rnd(layer.norm2_b, -0.1, 0.1)
            if isinstance(layer.mlp, RoutedExperts):
                rnd(layer.mlp.router, -0.5, 0.5)
                rnd(layer.mlp.correction, -0.3, 0.3)

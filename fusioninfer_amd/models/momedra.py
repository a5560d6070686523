"""Momedra: a decoder-only design of parallel-residual layers with a
repeated span.

Every layer norms the fp32 residual stream once and feeds a mixer and a
feed-forward side by side, x <- x + m (mixer(h) + ff(h)). The mixer is a
grouped-query attention with normed heads, a query temperature and a
per-head output gate (``attention``), an attention over cached low-rank
latents with a shared rotated key part and a softmax sink
(``latent_attention``), or a real-gated linear recurrence behind a short
convolution (``rglru``). The feed-forward is dense (squared relu) or a
mixture of experts with a shared expert. A span of layers may run several
times in a row with the same weights; each pass has its own cache and
state and is entered through a projection of [x; embedding output].

This module only ASSEMBLES the design from the reusable blocks in
``models/mixers.py``: it parses ``config.json`` (layer list, loop, sizes,
constants), declares what cache/state every layer RUN needs, and maps
checkpoint tensor names onto the merged parameters. The engine's block
manager, state-slot manager, scheduler and sampler serve it like any other
model.
"""

from __future__ import annotations

import dataclasses
from typing import Dict, Iterable, List, Optional, Tuple, Union

import torch
import torch.nn as nn
import torch.nn.functional as F

from fusioninfer_amd.config import ModelConfig
from fusioninfer_amd.distributed import parallel_state as ps
from fusioninfer_amd.distributed.layers import ReplicatedLinear
from fusioninfer_amd.models.mixers import (
    LatentAttention,
    LatentAttentionConfig,
    ParallelResidualLayer,
    RGLRUConfig,
    RGLRUMixer,
    RoutedExperts,
    SquaredReluMLP,
    TemperedGatedAttention,
    TemperedGatedAttentionConfig,
)
from fusioninfer_amd.ops import seqmix

ARCHITECTURE = "Momedra"


@dataclasses.dataclass
class FeedForwardConfig:
    kind: str                       # dense | moe
    ff: int                         # dense: hidden size; moe: per expert
    experts: int = 0
    top: int = 0
    shared_ff: int = 0              # 0: no shared expert


@dataclasses.dataclass
class MomedraLayerConfig:
    kind: str                       # attention | latent_attention | rglru
    mixer: Union[TemperedGatedAttentionConfig, LatentAttentionConfig,
                 RGLRUConfig]
    mlp: Optional[FeedForwardConfig]


@dataclasses.dataclass
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclasses.dataclass
class MomedraConfig:
    width: int
    vocab: int
    eps: float
    residual_mult: float
    layers: List[MomedraLayerConfig]
    loop: Optional[LoopConfig]

    def runs(self) -> List[Tuple[int, bool]]:
        """(layer index, enters a pass of the repeated span) in execution
        order."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        a, b, times = self.loop.start, self.loop.stop, self.loop.times
        out = [(i, False) for i in range(a)]
        for _ in range(times):
            out += [(i, i == a) for i in range(a, b)]
        out += [(i, False) for i in range(b, n)]
        return out


def _parse_mlp(i: int, mlp: Optional[dict]) -> Optional[FeedForwardConfig]:
    if not mlp:
        return None
    kind = mlp.get("kind")
    if kind == "dense":
        return FeedForwardConfig("dense", int(mlp["ff"]))
    if kind == "moe":
        r = mlp["router"]
        shared = mlp.get("shared") or {}
        return FeedForwardConfig(
            "moe", int(mlp["expert"]["ff"]), experts=int(r["experts"]),
            top=int(r["top"]), shared_ff=int(shared.get("ff", 0)))
    raise ValueError(f"layer {i}: unknown mlp kind {kind!r}")


def parse_config(raw: dict) -> MomedraConfig:
    """config.json -> MomedraConfig; every size and constant is read from
    the config."""
    layers = []
    for i, L in enumerate(raw["layers"]):
        kind, m = L.get("type"), L["mixer"]
        if kind == "attention":
            qt = m.get("q_temp") or {}
            mixer = TemperedGatedAttentionConfig(
                heads=int(m["heads"]),
                kv_heads=int(m.get("kv_heads", m["heads"])),
                dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                scale=float(m["scale"]),
                temp_coef=float(qt.get("coef", 0.0)),
                temp_every=int(qt.get("every", 0)))
        elif kind == "latent_attention":
            rot = m.get("rot") or {}
            rot_dim = int(m["rot_dim"])
            mixer = LatentAttentionConfig(
                heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim,
                vdim=int(m.get("vdim", m["dim"])), rank=int(m["kv_rank"]),
                scale=float(m["scale"]), rot_base=float(rot["base"]),
                rot_dims=int(rot.get("dims", rot_dim)))
        elif kind == "rglru":
            mixer = RGLRUConfig(width=int(m["width"]),
                                blocks=int(m.get("blocks", 1)),
                                conv=int(m.get("conv", 1)))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        layers.append(MomedraLayerConfig(kind, mixer,
                                         _parse_mlp(i, L.get("mlp"))))
    loop = None
    lp = raw.get("loop")
    if lp:
        loop = LoopConfig(int(lp["start"]), int(lp["stop"]),
                          int(lp.get("times", 1)))
        if not 0 <= loop.start < loop.stop <= len(layers) or loop.times < 1:
            raise ValueError(f"loop {lp} does not fit {len(layers)} layers")
    return MomedraConfig(
        width=int(raw["width"]), vocab=int(raw["vocab"]),
        eps=float(raw["norm"]["eps"]),
        residual_mult=float(raw.get("residual_mult", 1.0)),
        layers=layers, loop=loop)


def model_config_from_dict(raw: dict, model_path: Optional[str] = None,
                           name: str = ARCHITECTURE) -> ModelConfig:
    """Engine-level ModelConfig for a Momedra config dict (the registry's
    architecture hook)."""
    arch = parse_config(raw)
    heads, kv_heads, dim = 1, 1, arch.width
    for L in arch.layers:
        if L.kind == "attention":
            heads, kv_heads, dim = (L.mixer.heads, L.mixer.kv_heads,
                                    L.mixer.dim)
            break
        if L.kind == "latent_attention":
            heads, kv_heads, dim = (L.mixer.heads, 1,
                                    L.mixer.rank + L.mixer.rot_dim)
    ffs = [L.mlp for L in arch.layers if L.mlp is not None]
    return ModelConfig(
        name=name,
        architecture=ARCHITECTURE,
        arch=arch,
        hidden_size=arch.width,
        num_layers=len(arch.runs()),
        num_heads=heads,
        num_kv_heads=kv_heads,
        head_dim=dim,
        intermediate_size=max((f.ff for f in ffs), default=0),
        vocab_size=arch.vocab,
        rms_norm_eps=arch.eps,
        qk_norm=False,
        model_path=model_path,
        max_position_embeddings=1 << 24,
    )


class MomedraLM(nn.Module):
    """embedding -> parallel-residual layer runs -> final layer norm ->
    head.

    Engine interface (same as CausalLM): ``forward(ids, meta, caches)``
    returns the final-normed hidden rows, ``compute_logits`` applies the
    head. ``allocate_caches`` hands out one cache dict per layer RUN (a
    layer of the repeated span owns one per pass) and ``uses_state_slots``
    makes the runner build sequence-grouped metadata and the scheduler
    hand out state slots."""

    uses_state_slots = True
    supports_prefix_caching = False   # recurrent state has no block form

    def __init__(self, cfg: ModelConfig):
        super().__init__()
        assert ps.tp_world_size() == 1 and ps.pp_world_size() == 1, (
            "Momedra runs single-rank (TP/PP sharding of its mixers is "
            "not implemented)")
        self.cfg = cfg
        arch: MomedraConfig = cfg.arch
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
        self.loop_in = (ReplicatedLinear(2 * W, W, dtype=dtype)
                        if arch.loop is not None else None)
        layers = []
        for i, L in enumerate(arch.layers):
            torch.manual_seed(base_seed + 1000003 * (i + 2))
            if L.kind == "attention":
                mixer = TemperedGatedAttention(L.mixer, W, arch.eps, dtype)
            elif L.kind == "latent_attention":
                mixer = LatentAttention(L.mixer, W, arch.eps, dtype)
            else:
                mixer = RGLRUMixer(L.mixer, W, arch.eps, dtype)
            dense = routed = None
            if L.mlp is not None and L.mlp.kind == "dense":
                dense = SquaredReluMLP(W, L.mlp.ff, dtype, own_up=False)
            elif L.mlp is not None:
                routed = RoutedExperts(
                    W, L.mlp.ff, L.mlp.experts, L.mlp.top, dtype,
                    score="softmax", renorm=True, act="relu_sq",
                    router_bias=True)
                if L.mlp.shared_ff:
                    dense = SquaredReluMLP(W, L.mlp.shared_ff, dtype,
                                           own_up=False)
            layers.append(ParallelResidualLayer(
                mixer, dense, routed, W, arch.eps, arch.residual_mult,
                dtype))
        self.layers = nn.ModuleList(layers)
        self.final_norm = nn.Parameter(torch.ones(W, dtype=torch.float32),
                                       requires_grad=False)
        torch.manual_seed(base_seed + 1000003 * (len(arch.layers) + 2))
        self.lm_head = ReplicatedLinear(W, arch.vocab, dtype=dtype)
        torch.manual_seed(base_seed + 777)
        self.runs = arch.runs()
        # when set to a list, forward appends the residual stream after
        # every layer run (debugging, layer-by-layer tests)
        self.residual_trace: Optional[list] = None

    # ------------------------------------------------------ engine hooks
    @property
    def num_local_layers(self) -> int:
        return len(self.runs)

    def kv_block_bytes(self, block_size: int) -> int:
        n = sum(self.layers[i].mixer.block_bytes(block_size)
                for i, _ in self.runs)
        return max(n, 1)     # a model of recurrent layers only pages nothing

    def allocate_caches(self, num_blocks: int, block_size: int,
                        num_slots: int, device) -> list:
        """One dict per layer run: the paged tensors of its attention
        (model dtype) or the fp32 slot states of its recurrence."""
        return [self.layers[i].mixer.state_tensors(
            num_blocks, block_size, num_slots, device) for i, _ in self.runs]

    # ----------------------------------------------------------- forward
    def forward(self, input_ids, meta, caches, hidden=None, residual=None):
        eps = self.arch.eps
        x0 = self.embed_tokens[input_ids].contiguous()
        n = len(self.runs)
        # the stream starts as an fp32 copy of the embedding output (which
        # is read again at every pass entry), fused with the first norm
        # unless the first run enters a pass
        first = self.layers[self.runs[0][0]]
        resid, h = seqmix.cast_layer_norm(
            x0, None if self.runs[0][1] else first.norm1, eps)
        for r, ((i, enters), cache) in enumerate(zip(self.runs, caches)):
            layer = self.layers[i]
            if enters:
                # x <- W_in [x; embedding output], then this layer's norm
                xin = seqmix.concat_cast(resid, x0)
                resid, h = seqmix.cast_layer_norm(self.loop_in(xin),
                                                  layer.norm1, eps)
            if r + 1 == n:
                nxt = self.final_norm
            elif self.runs[r + 1][1]:
                nxt = None          # a pass entry rewrites x before its norm
            else:
                nxt = self.layers[self.runs[r + 1][0]].norm1
            h = layer(resid, h, meta, cache, nxt)
            if self.residual_trace is not None:
                self.residual_trace.append(resid.detach().clone())
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.lm_head(hidden).float()

    # ----------------------------------------------------------- weights
    def load_weights(self, tensors: Iterable[Tuple[str, torch.Tensor]]) -> int:
        """Checkpoint names -> parameters. A layer's input branches (the
        mixer's, the dense or shared up projection) land in its merged
        projection, expert matrices in the stacked expert tensors, the
        recurrence's gate blocks in one stacked fp32 tensor; gains, biases
        of gates, sinks and decays are kept in fp32."""
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
            if layer.routed is not None:
                layer.routed.invalidate_packed()
        return n

    def expected_tensor_names(self) -> List[str]:
        return list(self._name_map())

    def _name_map(self) -> Dict[str, tuple]:
        """checkpoint name -> (parameter, view spec or None)."""
        out: Dict[str, tuple] = {
            "embed": (self.embed_tokens, None),
            "head": (self.lm_head.weight, None),
            "final.norm": (self.final_norm, None),
        }
        if self.loop_in is not None:
            out["loop.in"] = (self.loop_in.weight, None)
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            mp = p + "mix."
            mod = layer.mixer
            out[p + "norm1"] = (layer.norm1, None)
            for br in mod.in_names:
                rows = layer.in_proj_rows(br)
                out[mp + br] = (layer.in_proj.weight, rows)
                if mod.has_bias and br in mod.biased:
                    out[mp + br + ".b"] = (layer.in_proj.bias, rows)
            out[mp + "o"] = (mod.o_proj.weight, None)
            if isinstance(mod, TemperedGatedAttention):
                out[mp + "q.norm"] = (mod.q_norm, None)
                out[mp + "k.norm"] = (mod.k_norm, None)
            elif isinstance(mod, LatentAttention):
                out[mp + "dkv.norm"] = (mod.c_norm, None)
                out[mp + "uk"] = (mod.uk, None)
                out[mp + "uv"] = (mod.uv, None)
                if mod.sink is not None:
                    out[mp + "sink"] = (mod.sink, None)
            else:
                bw = mod.cfg.width // mod.cfg.blocks
                out[mp + "conv"] = (mod.conv_w, None)
                out[mp + "conv.b"] = (mod.conv_b, None)
                out[mp + "ra"] = (mod.gate_w, ("cols", 0, bw))
                out[mp + "ri"] = (mod.gate_w, ("cols", bw, bw))
                out[mp + "ra.b"] = (mod.gate_b, ("cols", 0, bw))
                out[mp + "ri.b"] = (mod.gate_b, ("cols", bw, bw))
                out[mp + "lam"] = (mod.lam, None)
            fp = p + "mlp."
            if layer.routed is not None:
                out[fp + "router"] = (layer.routed.router, None)
                out[fp + "router.b"] = (layer.routed.router_bias, None)
                for e in range(layer.routed.experts):
                    out[f"{fp}e{e}.up"] = (layer.routed.gate_up, ("idx", e))
                    out[f"{fp}e{e}.down"] = (layer.routed.down, ("idx", e))
                if layer.dense is not None:
                    out[fp + "shared.up"] = (layer.in_proj.weight,
                                             layer.in_proj_rows("up"))
                    out[fp + "shared.down"] = (
                        layer.dense.down_proj.weight, None)
            elif layer.dense is not None:
                out[fp + "up"] = (layer.in_proj.weight,
                                  layer.in_proj_rows("up"))
                out[fp + "down"] = (layer.dense.down_proj.weight, None)
        return out

    @staticmethod
    def _view(param, spec):
        dst = param.data
        if spec is None:
            return dst
        if spec[0] == "cols":        # [B, a:a+n, ...] of a stacked tensor
            return dst[:, spec[1]: spec[1] + spec[2]]
        if spec[0] == "idx":
            return dst[spec[1]]
        return dst[spec[0]: spec[0] + spec[1]]

    def _load_one(self, name: str, t: torch.Tensor) -> None:
        names = getattr(self, "_names", None)
        if names is None:
            names = self._names = self._name_map()
        if name not in names:
            if name == "loop.in" and self.loop_in is None:
                return      # no repeated span configured: nothing enters it
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
        """Random-init use (benchmarks, tests): give gains, biases, sinks,
        decays and convolutions non-trivial values so every branch
        contributes."""
        g = torch.Generator().manual_seed(seed)

        def rnd(p, lo, hi):
            p.data.copy_((torch.rand(p.shape, generator=g) * (hi - lo) + lo)
                         .to(device=p.device, dtype=p.dtype))

        rnd(self.final_norm, 0.8, 1.2)
        for layer in self.layers:
            rnd(layer.norm1, 0.5, 1.5)
            mod = layer.mixer
            if layer.in_proj.bias is not None:
                rnd(layer.in_proj.bias, -0.1, 0.1)
                for br in layer.branches:
                    if br not in getattr(mod, "biased", ()):
                        a, n = layer.in_proj_rows(br)
                        layer.in_proj.bias.data[a: a + n] = 0
            if layer.routed is not None:
                rnd(layer.routed.router, -0.5, 0.5)
                rnd(layer.routed.router_bias, -0.5, 0.5)
            if isinstance(mod, TemperedGatedAttention):
                rnd(mod.q_norm, 0.5, 1.5)
                rnd(mod.k_norm, 0.5, 1.5)
            elif isinstance(mod, LatentAttention):
                rnd(mod.c_norm, 0.5, 1.5)
                if mod.sink is not None:
                    rnd(mod.sink, -1.0, 2.0)
            else:
                rnd(mod.conv_w, -0.5, 0.5)
                rnd(mod.conv_b, -0.1, 0.1)
                rnd(mod.gate_b, -1.0, 1.0)
                rnd(mod.lam, -3.0, 1.0)

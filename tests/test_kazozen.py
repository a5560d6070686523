"""Kazozen through the engine against the float64 oracle in
tests/oracles/kazozen_oracle.py: every mechanism alone, prompts against
token-by-token decoding, portions down to two tokens, unequal batches,
recycled pages and slots, far keys and window/kept-key/page/tile/span
borders, first tokens, long decoding, odd sizes, and greedy generation
through the scheduler.

The same cases run on the CPU ops (always) and on the HIP kernels (gpu
marker)."""

import json
import math
import os
import subprocess
import sys

import pytest
import torch

from fusioninfer_amd import ops
from fusioninfer_amd.config import CacheConfig, EngineConfig, SchedulerConfig
from fusioninfer_amd.engine.llm_engine import LLMEngine
from fusioninfer_amd.engine.sequence import SamplingParams
from fusioninfer_amd.models import registry
from fusioninfer_amd.models.mixers import RoutedExperts
from fusioninfer_amd.ops import seqmix
from tests.oracles import kazozen_oracle as oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64
TOL = 2e-4   # fp32 engine vs float64 oracle, relative
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---------------------------------------------------------------- configs

def rot_cfg(dims, base=500.0, scaling=True, factor=4.0, original=64,
            fast=8.0, slow=2.0):
    r = {"dims": dims, "base": base}
    if scaling:
        r["scaling"] = {"factor": factor, "original": original, "fast": fast,
                        "slow": slow}
    return r


def mixer_cfg(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.3, window=13,
              keep=3, rot=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": scale}
    if window:
        m["mask"] = {"size": window, "keep_first": keep}
    if rot is not None:
        m["rot"] = rot
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def dense_cfg(ff=40, limit=1.2):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe_cfg(ff=24, experts=6, top=2, count=3, keep=2, limit=0.9):
    r = {"experts": experts, "top": top}
    if count:
        r["groups"] = {"count": count, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}


def layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def small_config():
    """Sizes chosen so that nothing coincides: key and value sizes differ,
    grouped heads, partial rotation, windows that are no multiple of the
    page size, layers that borrow keys and values (one across another
    owner), a layer without a window, one without feed-forward."""
    r0, r2 = rot_cfg(6), rot_cfg(12, base=90.0, scaling=False)
    return {
        "architecture": "Kazozen",
        "vocab": 89,
        "width": 48,
        "norm": {"eps": 1e-3},
        "embedding": {"scale": 3.0, "bigram": {"buckets": 37, "mul_prev": 11,
                                               "mul_cur": 5}},
        "logit_softcap": 9.0,
        "layers": [
            layer(mixer_cfg(rot=r0), dense_cfg()),
            layer(mixer_cfg(scale=0.2, window=7, keep=0, rot=r0, kv_from=0),
                  moe_cfg()),
            layer(mixer_cfg(heads=3, kv_heads=1, dim=12, vdim=4, scale=0.11,
                            window=0, rot=r2), None),
            layer(mixer_cfg(heads=3, kv_heads=1, dim=12, vdim=4, scale=0.4,
                            window=20, keep=5, rot=r2, kv_from=2),
                  moe_cfg(ff=16, experts=4, top=2, count=2, keep=1)),
            layer(mixer_cfg(window=30, keep=1, rot=r0, kv_from=0),
                  dense_cfg(24, 0.7)),
        ],
    }


def make_engine(raw, device, dtype="float32", blocks=64, max_seqs=4,
                seed=0, budget=4096, eager=True):
    mc = registry.model_config_from_dict(raw)
    mc.dtype = dtype
    cfg = EngineConfig(
        model=mc,
        cache=CacheConfig(num_gpu_blocks=blocks, enable_prefix_caching=False),
        scheduler=SchedulerConfig(max_num_seqs=max_seqs,
                                  max_num_batched_tokens=budget,
                                  max_model_len=blocks * 16,
                                  prefill_admission_tokens=0),
        enforce_eager=eager,
        num_state_slots=max_seqs,
        seed=seed,
    )
    eng = LLMEngine(cfg, device=device)
    model = eng.runner.model
    # livelier weights than the 0.02-std init so that every branch matters
    g = torch.Generator().manual_seed(seed + 2)
    for name, p in model.named_parameters():
        if p.dim() >= 2:
            p.data.copy_((torch.randn(p.shape, generator=g)
                          / math.sqrt(p.shape[-1])).to(p.dtype).to(p.device))
    model.randomize_small_params(seed + 1)
    for lay in model.layers:
        if isinstance(lay.mlp, RoutedExperts):
            lay.mlp.invalidate_packed()
    W = {k: v.detach().cpu().to(F64)
         for k, v in model.export_weights().items()}
    return eng, W


def rel_err(got, want):
    """Mean-free RMS difference relative to the RMS of the expected row."""
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()).max().item()


def run_schedule(eng, steps):
    """steps: [[(id, tokens, want)], ...] with ('end', id) tuples allowed;
    returns {id: {position: logits}}."""
    got, at = {}, {}
    for step in steps:
        entries = [e for e in step if e[0] != "end"]
        end = [e[1] for e in step if e[0] == "end"]
        out = eng.forced_step(entries, end).cpu()
        row = 0
        for rid, toks, want in entries:
            for w in want:
                got.setdefault(rid, {})[at.get(rid, 0) + w] = out[row]
                row += 1
            at[rid] = at.get(rid, 0) + len(toks)
        for rid in end:
            at.pop(rid, None)
    return got


def tokens(n, seed, vocab=89):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def mk(v, device):
    return torch.tensor(v, dtype=torch.int32, device=device)


# ----------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("pair", [True, False])
@pytest.mark.parametrize("W", [20, 21])
def test_pair_embedding_and_previous_token_state(device, pair, W):
    g = torch.Generator().manual_seed(3)
    V, B = 23, 7
    emb = torch.randn(V, W, generator=g)
    tab = torch.randn(B + 1, W, generator=g) if pair else None
    bg = {"buckets": B, "mul_prev": 5, "mul_cur": 3}
    cfg = {"embedding": {"scale": 2.5, "bigram": bg if pair else None}}
    Wt = {"embed": emb.to(F64)}
    if pair:
        Wt["bigram"] = tab.to(F64)
    seqs = {0: tokens(9, 1, V), 1: tokens(4, 2, V), 2: tokens(6, 3, V)}
    want = {s: oracle.embed_tokens(t, Wt, cfg) for s, t in seqs.items()}
    # stale ids of earlier owners in every slot
    state = mk([17, 3, 11, 5], device)
    # (sequence, first position, rows) with slots 2, 0, 3
    slot = {0: 2, 1: 0, 2: 3}
    steps = [[(0, 0, 5), (1, 0, 1)], [(0, 5, 1), (1, 1, 2), (2, 0, 6)],
             [(0, 6, 3), (1, 3, 1)]]
    for step in steps:
        ids = sum((seqs[s][p0:p0 + n] for s, p0, n in step), [])
        pos = sum((list(range(p0, p0 + n)) for s, p0, n in step), [])
        cu = [0]
        for _, _, n in step:
            cu.append(cu[-1] + n)
        row_seq = sum(([i] * n for i, (_, _, n) in enumerate(step)), [])
        resid, act = seqmix.pair_embed(
            torch.tensor(ids, dtype=torch.long, device=device),
            emb.to(device), 2.5, tab.to(device) if pair else None, B, 5, 3,
            state, mk(cu, device), mk(row_seq, device),
            mk([slot[s] for s, _, _ in step], device), mk(pos, device),
            torch.float32)
        a = 0
        for s, p0, n in step:
            assert torch.allclose(resid[a:a + n].cpu().double(),
                                  want[s][p0:p0 + n], atol=1e-5)
            a += n
        assert torch.equal(act.cpu(), resid.cpu())
    # a slot that ended with some id serves a new sequence from position 0
    assert state.tolist()[2] == seqs[0][8]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T,W", [(5, 24), (3, 101), (4, 1024), (2, 2052),
                                 (2, 4100), (1, 9000)])
def test_post_norm_residual_and_affine_norm(device, T, W):
    g = torch.Generator().manual_seed(W)
    y = torch.randn(T, W, generator=g) * 3 + 1.5
    x = torch.randn(T, W, generator=g)
    w = torch.rand(W, generator=g) + 0.5
    b = torch.randn(W, generator=g) * 0.1
    want = x.double() + oracle.layer_norm_wb(y.double(), w.double(),
                                             b.double(), 1e-3)
    resid = x.clone().to(device)
    out = seqmix.post_norm_residual_(resid, y.to(device), w.to(device),
                                     b.to(device), 1e-3, torch.float32)
    assert torch.allclose(resid.cpu().double(), want, atol=2e-5)
    assert torch.allclose(out.cpu().double(), want, atol=2e-5)
    n = seqmix.layer_norm_affine(x.to(device), w.to(device), b.to(device),
                                 1e-3, torch.float32)
    assert torch.allclose(
        n.cpu().double(),
        oracle.layer_norm_wb(x.double(), w.double(), b.double(), 1e-3),
        atol=2e-5)
    # bf16 activations: the stream stays fp32, only the copy is rounded
    resid = x.clone().to(device)
    yb = y.to(torch.bfloat16)
    out = seqmix.post_norm_residual_(resid, yb.to(device), w.to(device),
                                     b.to(device), 1e-3, torch.bfloat16)
    want = x.double() + oracle.layer_norm_wb(yb.double(), w.double(),
                                             b.double(), 1e-3)
    assert torch.allclose(resid.cpu().double(), want, atol=2e-5)
    assert torch.equal(out.cpu(), resid.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("rot", [
    rot_cfg(6), rot_cfg(48, base=1e5, factor=3.0, original=1024, fast=16.0,
                        slow=2.0),
    rot_cfg(16, base=100.0, factor=8.0, original=30, fast=2.0, slow=1.9),
    rot_cfg(32, base=10000.0, factor=1.5, original=4096, fast=1e6, slow=1e5),
    rot_cfg(8, scaling=False)])
def test_blended_frequencies(rot):
    sc = rot.get("scaling") or {}
    f, mult = seqmix.blended_rotary(
        rot["dims"], rot["base"], sc.get("factor", 1.0),
        sc.get("original", 0.0), sc.get("fast", 0.0), sc.get("slow", 0.0))
    wf, wm = oracle.rotary_frequencies(rot)
    assert torch.allclose(f.double(), torch.tensor(wf, dtype=F64), rtol=1e-6)
    assert abs(mult - wm) < 1e-12


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,V,dims,own", [
    (4, 2, 8, 12, 6, True), (3, 1, 12, 4, 12, True), (5, 5, 7, 3, 4, True),
    (2, 1, 64, 64, 32, True), (4, 2, 8, 12, 0, True), (6, 2, 10, 5, 10, False)])
def test_whole_projection_norm_rotation_and_cache(device, H, G, D, V, dims,
                                                  own):
    g = torch.Generator().manual_seed(H * 100 + D)
    Wd, T, eps, bs = 20, 9, 1e-3, 16
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V}
    if dims:
        m["rot"] = rot_cfg(dims)
    Wt = {"q": torch.randn(H * D, Wd, generator=g),
          "q.b": torch.randn(H * D, generator=g),
          "k": torch.randn(G * D, Wd, generator=g),
          "k.b": torch.randn(G * D, generator=g),
          "v": torch.randn(G * V, Wd, generator=g),
          "v.b": torch.randn(G * V, generator=g),
          "q.norm": torch.rand(H * D, generator=g) + 0.5,
          "k.norm": torch.rand(G * D, generator=g) + 0.5}
    Wt = {k: v.to(F64) for k, v in Wt.items()}
    h = torch.randn(T, Wd, generator=g).to(F64)
    pos0 = 37
    q_want = oracle.queries(h, Wt, "", m, eps, pos0)
    k_want, v_want = oracle.keys_values(h, Wt, "", m, eps, pos0)
    # one merged projection output, branches as column slices
    proj = torch.cat([h @ Wt["q"].T + Wt["q.b"], h @ Wt["k"].T + Wt["k.b"],
                      h @ Wt["v"].T + Wt["v.b"]], dim=1).float().to(device)
    q, k, v = proj.split([H * D, G * D, G * V], dim=1)
    kc = torch.full((6, G, bs, D), 7.0, device=device)
    vc = torch.full((6, G, bs, V), 7.0, device=device)
    pages = [4, 1, 5, 0]
    pos = list(range(pos0, pos0 + T))
    slots = [pages[p // bs] * bs + p % bs for p in pos]
    slots[2] = -1     # a padding row writes nothing
    if dims:
        f, mult = seqmix.blended_rotary(dims, 500.0, 4.0, 64, 8.0, 2.0)
    else:
        f, mult = torch.zeros(0), 1.0
    qn = seqmix.widenorm_rope_cache_(
        q, k if own else None, v if own else None, mk(pos, device),
        Wt["q.norm"].float().to(device),
        Wt["k.norm"].float().to(device) if own else None, eps, f.to(device),
        mult, kc, vc, mk(slots, device), H, G, D, V)
    assert torch.allclose(qn.cpu().double(), q_want, atol=2e-5)
    for r, p in enumerate(pos):
        got_k = kc[pages[p // bs], :, p % bs].cpu().double()
        got_v = vc[pages[p // bs], :, p % bs].cpu().double()
        if own and r != 2:
            assert torch.allclose(got_k, k_want[r], atol=2e-5)
            assert torch.allclose(got_v, v_want[r], atol=2e-5)
        else:
            assert (got_k == 7.0).all() and (got_v == 7.0).all()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T,F,limit", [(3, 10, 0.5), (5, 64, 7.0),
                                       (2, 1030, 1.5)])
def test_clamped_unit_and_logit_cap(device, T, F, limit):
    g = torch.Generator().manual_seed(F)
    gu = torch.randn(T, 2 * F, generator=g) * 3
    want = oracle.clamped_glu(gu[:, :F].double(), gu[:, F:].double(), limit)
    got = seqmix.clamped_glu(gu.to(device), limit)
    assert torch.allclose(got.cpu().double(), want, atol=1e-5)
    wide = torch.randn(T, 3 * F, generator=g).to(device) * 3
    got = seqmix.clamped_glu(wide[:, F:], limit)      # strided rows
    w = wide.cpu().double()
    assert torch.allclose(
        got.cpu().double(),
        oracle.clamped_glu(w[:, F:2 * F], w[:, 2 * F:], limit), atol=1e-5)
    z = torch.randn(T, F, generator=g) * 20
    got = seqmix.tanh_cap_(z.clone().to(device), 4.0)
    assert torch.allclose(got.cpu().double(),
                          4.0 * torch.tanh(z.double() / 4.0), atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,count,keep", [
    (8, 2, 4, 3), (6, 2, 3, 2), (4, 2, 2, 1), (12, 5, 3, 2), (5, 2, 5, 3),
    (9, 3, 1, 1), (16, 4, 4, 4), (130, 8, 10, 3), (7, 7, 1, 1), (64, 1, 8, 1)])
def test_group_limited_router(device, E, top, count, keep):
    g = torch.Generator().manual_seed(E * 7 + top)
    T = 33
    z = torch.randn(T, E, generator=g) * 2
    # corrections large enough to change the choice and to make choice
    # scores negative
    corr = torch.randn(E, generator=g) * 0.8 - 0.6
    topv, topi = ops.moe_route_grouped(z.to(device), corr.to(device), top,
                                       count, keep)
    r = {"experts": E, "top": top, "groups": {"count": count, "keep": keep}}
    for t in range(T):
        want = oracle.route(z[t].double(), corr.double(), r)
        assert topi[t].tolist() == [e for e, _ in want], t
        assert torch.allclose(topv[t].cpu().double(),
                              torch.stack([w for _, w in want]), atol=1e-6)


def _experts_case(device, dtype, width, ff, E, top, count, keep, T, limit,
                  seed=0):
    torch.manual_seed(seed)
    mod = RoutedExperts(width, ff, E, top, dtype, score="sigmoid",
                        renorm=False, act="clamped_glu", limit=limit,
                        groups=(count, keep))
    g = torch.Generator().manual_seed(seed + 1)
    for p in (mod.gate_up, mod.down):
        p.data.copy_((torch.randn(p.shape, generator=g)
                      / math.sqrt(p.shape[-1])).to(dtype))
    mod.router.data.copy_(torch.randn(E, width, generator=g) * 0.4)
    mod.correction.data.copy_(torch.randn(E, generator=g) * 0.3)
    x = (torch.randn(T, width, generator=g)).to(dtype)
    Wt = {"router": mod.router.data.double(),
          "correction": mod.correction.data.double()}
    for e in range(E):
        Wt[f"e{e}.gate"] = mod.gate_up.data[e, :ff].double()
        Wt[f"e{e}.up"] = mod.gate_up.data[e, ff:].double()
        Wt[f"e{e}.down"] = mod.down.data[e].double()
    mlp = {"expert": {"ff": ff, "limit": limit},
           "router": {"experts": E, "top": top,
                      "groups": {"count": count, "keep": keep}}}
    want = oracle.routed_experts(x.double(), Wt, "", mlp)
    got = mod.to(device)(x.to(device))
    return got.cpu().double(), want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("width,ff,E,top,count,keep,T", [
    (48, 24, 6, 2, 3, 2, 19), (20, 7, 5, 5, 1, 1, 4), (33, 65, 8, 1, 8, 2, 70),
    (16, 16, 1, 1, 1, 1, 3)])
def test_clamped_experts_fp32(device, width, ff, E, top, count, keep, T):
    got, want = _experts_case(device, torch.float32, width, ff, E, top, count,
                              keep, T, limit=0.8)
    assert rel_err(got, want) < TOL


@pytest.mark.gpu
@pytest.mark.parametrize("width,ff,E,top,count,keep,T", [
    (128, 64, 8, 2, 4, 3, 40),      # MFMA kernel, 16-row tiles
    (256, 128, 4, 2, 2, 1, 600),    # MFMA kernel, 128-row tiles
    (96, 48, 6, 2, 3, 2, 50)])      # sizes the tiles do not divide
def test_clamped_experts_bf16_gpu(width, ff, E, top, count, keep, T):
    got, want = _experts_case("cuda", torch.bfloat16, width, ff, E, top,
                              count, keep, T, limit=1.1)
    assert rel_err(got, want) < 3e-2


# ------------------------------------------- attention on crafted inputs

def _crafted_attention(device, H, G, DK, DV, ctx, hot, rows, window, keep,
                       dtype=torch.float32, seed=0, gate=True):
    """One sequence of ctx keys in shuffled pages; the last `rows`
    positions are the query rows. Key `hot` and all queries share a strong
    direction, so if `hot` is visible it takes nearly all the weight and
    if it is hidden the result is something else entirely."""
    g = torch.Generator().manual_seed(seed + hot + 1000 * rows)
    bs = 16
    nb = (ctx + bs - 1) // bs
    q = torch.randn(rows, H, DK, generator=g) * 0.3
    k = torch.randn(ctx, G, DK, generator=g) * 0.3
    v = torch.randn(ctx, G, DV, generator=g)
    u = torch.randn(DK, generator=g)
    u = u / u.norm()
    k[hot] += 4.0 * u
    q += 4.0 * u
    sink = torch.randn(H, generator=g)
    gt = torch.randn(rows, H * DV, generator=g)
    pages = torch.randperm(nb + 3, generator=g)[:nb].tolist()
    kc = torch.zeros(nb + 3, G, bs, DK)
    vc = torch.zeros(nb + 3, G, bs, DV)
    for j in range(ctx):
        kc[pages[j // bs], :, j % bs] = k[j]
        vc[pages[j // bs], :, j % bs] = v[j]
    q, kc, vc, gt = (t.to(dtype) for t in (q, kc, vc, gt))
    pos = list(range(ctx - rows, ctx))
    tiles = (seqmix.build_attention_tiles([rows], device=device)
             if rows > 1 else None)
    out = seqmix.sink_paged_attention(
        q.to(device), kc.to(device), vc.to(device), mk([pages], device),
        mk([0] * rows, device), mk(pos, device), 0.9, sink=sink.to(device),
        out_gate=gt.to(device) if gate else None,
        seq_cu=mk([0, rows], device), tiles=tiles, window=window,
        keep_first=keep)
    mask = {"size": window, "keep_first": keep} if window else None
    kd = torch.stack([kc[pages[j // bs], :, j % bs] for j in range(ctx)])
    vd = torch.stack([vc[pages[j // bs], :, j % bs] for j in range(ctx)])
    want = torch.stack([
        oracle.attend_row(q[r].double(), kd.double(), vd.double(), pos[r],
                          mask, 0.9, sink.double()) for r in range(rows)])
    if gate:
        want = want * torch.sigmoid(gt.double()).reshape(rows, H, DV)
    return out.cpu().double(), want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("rows", [1, 2, 43])
@pytest.mark.parametrize("back", ["in", "out", "kept", "dropped", "far"])
def test_window_and_kept_key_edges(device, rows, back):
    """The strong key sits just inside / just outside the LAST row's
    window, is the last kept first key / the first one not kept, or lies
    hundreds of positions back without a window."""
    ctx, window, keep = 330, 50, 6
    hot = {"in": ctx - window, "out": ctx - 1 - window, "kept": keep - 1,
           "dropped": keep, "far": 2}[back]
    if back == "far":
        window = keep = 0
    got, want = _crafted_attention(device, 4, 2, 8, 12, ctx, hot, rows,
                                   window, keep)
    assert rel_err(got.reshape(rows, -1), want.reshape(rows, -1)) < TOL


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("hot", [0, 15, 16, 63, 64, 127, 128, 255, 256, 298])
@pytest.mark.parametrize("rows", [1, 2, 43])
def test_strong_key_at_page_tile_and_span_borders(device, hot, rows):
    # beyond position 99 the strong key is the oldest one the last row's
    # window still holds
    got, want = _crafted_attention(device, 2, 1, 16, 16, 300, hot, rows,
                                   window=300 - hot if hot > 99 else 0,
                                   keep=0)
    assert rel_err(got.reshape(rows, -1), want.reshape(rows, -1)) < TOL


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("rows,ctx,window,keep,hot", [
    (200, 900, 72, 7, 6), (200, 900, 72, 7, 7), (200, 900, 72, 7, 828),
    (200, 900, 72, 7, 827), (130, 700, 64, 0, 636), (130, 700, 64, 70, 69),
    (130, 700, 64, 70, 70), (1, 900, 72, 7, 6), (1, 900, 72, 7, 7),
    (1, 900, 300, 260, 259), (1, 900, 300, 260, 600), (1, 900, 300, 260, 599),
    (64, 1100, 0, 0, 3)])
def test_tiled_sizes_skip_hidden_tiles_and_spans(dtype, D, rows, ctx, window,
                                                 keep, hot):
    """Head sizes with an MFMA tile kernel; contexts long enough that whole
    key tiles and whole 256-key spans lie between the kept first keys and
    the window."""
    got, want = _crafted_attention("cuda", 4, 2, D, D, ctx, hot, rows, window,
                                   keep, dtype=dtype)
    tol = TOL if dtype == torch.float32 else 3e-2
    assert rel_err(got.reshape(rows, -1), want.reshape(rows, -1)) < tol


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,DK,DV", [(1, 1, 7, 5), (10, 1, 24, 8),
                                       (12, 3, 36, 130), (2, 2, 130, 20)])
def test_attention_sizes_and_head_batches(device, H, G, DK, DV):
    for rows in (1, 5):
        got, want = _crafted_attention(device, H, G, DK, DV, 70, 30, rows,
                                       window=45, keep=2, gate=rows == 1)
        assert rel_err(got.reshape(rows, -1), want.reshape(rows, -1)) < TOL


@pytest.mark.parametrize("device", DEVICES)
def test_large_sink_takes_the_weight(device):
    g = torch.Generator().manual_seed(5)
    H, D = 2, 8
    q = torch.randn(1, H, D, generator=g)
    kc = torch.randn(1, 1, 16, D, generator=g)
    vc = torch.randn(1, 1, 16, D, generator=g)
    sink = torch.tensor([30.0, -30.0])
    out = seqmix.sink_paged_attention(
        q.to(device), kc.to(device), vc.to(device), mk([[0]], device),
        mk([0], device), mk([9], device), 0.5, sink=sink.to(device))
    want = oracle.attend_row(q[0].double(), kc[0].transpose(0, 1).double(),
                             vc[0].transpose(0, 1).double(), 9, None, 0.5,
                             sink.double())
    assert out[0, 0].abs().max() < 1e-6
    assert torch.allclose(out[0].cpu().double(), want, atol=1e-5)


# ------------------------------------------------------ through the engine

@pytest.fixture(scope="module", params=DEVICES)
def small(request):
    raw = small_config()
    eng, W = make_engine(raw, request.param)
    toks = tokens(70, 11)
    trace = []
    want = oracle.forward(toks, W, raw, trace)
    return raw, eng, W, toks, want, trace


def test_whole_prompt_layers_and_first_tokens(small):
    raw, eng, W, toks, want, layers = small
    model = eng.runner.model
    model.residual_trace = []
    got = run_schedule(eng, [[("a", toks, list(range(len(toks))))],
                             [("end", "a")]])
    trace, model.residual_trace = model.residual_trace, None
    rows = torch.stack([got["a"][p] for p in range(len(toks))])
    assert rel_err(rows, want) < TOL
    assert rel_err(rows[:3], want[:3]) < TOL
    assert len(trace) == len(layers) == len(raw["layers"])
    for got_x, want_x in zip(trace, layers):
        assert rel_err(got_x, want_x) < TOL
    one = run_schedule(eng, [[("b", toks[:1], [0])], [("end", "b")]])
    assert rel_err(one["b"][0][None], want[:1]) < TOL


def test_prefill_against_token_by_token_decoding(small):
    raw, eng, W, toks, want, _ = small
    steps = [[("d", toks[:1], [0])]]
    steps += [[("d", [t], [0])] for t in toks[1:]]
    steps.append([("end", "d")])
    got = run_schedule(eng, steps)
    rows = torch.stack([got["d"][p] for p in range(len(toks))])
    assert rel_err(rows, want) < TOL


@pytest.mark.parametrize("sizes", [[2] * 35, [3, 16, 1, 2, 31, 2, 15],
                                   [33, 2, 35], [64, 2, 2, 2]])
def test_portions_of_several_sizes(small, sizes):
    raw, eng, W, toks, want, _ = small
    assert sum(sizes) == len(toks)
    steps, a = [], 0
    for n in sizes:
        steps.append([("p", toks[a:a + n], list(range(n)))])
        a += n
    steps.append([("end", "p")])
    got = run_schedule(eng, steps)
    rows = torch.stack([got["p"][p] for p in range(len(toks))])
    assert rel_err(rows, want) < TOL


def test_unequal_batch_equals_each_alone_and_recycles(small):
    raw, eng, W, toks, want, _ = small
    reqs = {"r0": tokens(41, 1), "r1": tokens(5, 2), "r2": tokens(23, 3),
            "r3": tokens(1, 4), "r4": tokens(37, 5), "r5": tokens(18, 6)}
    ref = {k: oracle.forward(v, W, raw) for k, v in reqs.items()}
    all_ = lambda n: list(range(n))
    t = reqs
    steps = [
        [("r0", t["r0"][:7], all_(7)), ("r1", t["r1"][:2], all_(2))],
        [("r0", t["r0"][7:8], [0]), ("r1", t["r1"][2:], all_(3)),
         ("r2", t["r2"][:20], all_(20)), ("r3", t["r3"], [0]),
         ("end", "r1"), ("end", "r3")],
        # r4 and r5 take the slots and pages r1 and r3 gave back
        [("r4", t["r4"][:30], all_(30)), ("r0", t["r0"][8:9], [0]),
         ("r5", t["r5"][:1], [0]), ("r2", t["r2"][20:21], [0])],
        [("r5", t["r5"][1:2], [0]), ("r0", t["r0"][9:41], all_(32)),
         ("r2", t["r2"][21:], all_(2)), ("r4", t["r4"][30:31], [0]),
         ("end", "r0"), ("end", "r2")],
        [("r4", t["r4"][31:], all_(6)), ("r5", t["r5"][2:], all_(16)),
         ("end", "r4"), ("end", "r5")],
    ]
    free_before = (eng.block_manager.num_free(), eng.state_manager.num_free())
    got = run_schedule(eng, steps)
    for k, v in reqs.items():
        rows = torch.stack([got[k][p] for p in range(len(v))])
        assert rel_err(rows, ref[k]) < TOL, k
    assert (eng.block_manager.num_free(),
            eng.state_manager.num_free()) == free_before


def test_slot_and_pages_reused_by_a_shorter_request(small):
    """A long request leaves its last token and pages behind; the next one
    in the same slot and pages must start from nothing, and one that is
    left out of a step must find its previous token again."""
    raw, eng, W, toks, want, _ = small
    run_schedule(eng, [[("x", tokens(60, 9), [])], [("end", "x")]])
    got = run_schedule(eng, [[("y", toks[:2], [0, 1])],
                             [("z", tokens(5, 8), [])],
                             [("y", toks[2:9], list(range(7)))],
                             [("end", "y"), ("end", "z")]])
    rows = torch.stack([got["y"][p] for p in range(9)])
    assert rel_err(rows, want[:9]) < TOL


def test_greedy_generation_through_scheduler(small):
    raw, eng, W, toks, want, _ = small
    prompts = [toks[:13], toks[20:23], toks[30:51]]
    n_new = 12
    outs = eng.generate(prompts, SamplingParams(max_tokens=n_new))
    for p, o in zip(prompts, outs):
        assert o.output_token_ids == oracle.greedy(p, W, raw, n_new)
    assert eng.state_manager.num_free() == eng.state_manager.num_slots


def test_generation_with_small_token_budget_chunks_prompts():
    """The scheduler's own chunked prefill (budget 8 tokens a step) and
    more requests than slots."""
    raw = small_config()
    eng, W = make_engine(raw, "cpu", max_seqs=2, budget=8, seed=3)
    prompts = [tokens(21, 31), tokens(9, 32), tokens(14, 33)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=6))
    for p, o in zip(prompts, outs):
        assert o.output_token_ids == oracle.greedy(p, W, raw, 6)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_windows_pages_and_spans(device):
    r = rot_cfg(8, base=50.0, factor=3.0, original=40, fast=6.0, slow=1.5)
    raw = {
        "architecture": "Kazozen", "vocab": 50, "width": 32,
        "norm": {"eps": 1e-5},
        "embedding": {"scale": 1.5, "bigram": {"buckets": 19, "mul_prev": 7,
                                               "mul_cur": 13}},
        "logit_softcap": 20.0,
        "layers": [
            layer(mixer_cfg(heads=2, kv_heads=2, dim=16, vdim=16, scale=0.25,
                            window=40, keep=4, rot=r),
                  moe_cfg(ff=16, experts=4, top=2, count=2, keep=1)),
            layer(mixer_cfg(heads=2, kv_heads=2, dim=16, vdim=16, scale=0.3,
                            window=270, keep=0, rot=r, kv_from=0),
                  dense_cfg(16)),
        ],
    }
    eng, W = make_engine(raw, device, blocks=24)
    toks = tokens(300, 21, vocab=50)
    want = oracle.forward(toks, W, raw)
    steps = [[("a", toks[:10], list(range(10)))]]
    steps += [[("a", [t], [0])] for t in toks[10:]]
    got = run_schedule(eng, steps)
    rows = torch.stack([got["a"][p] for p in range(len(toks))])
    assert rel_err(rows, want) < TOL


@pytest.mark.parametrize("device", DEVICES)
def test_values_that_could_hide_faults(device):
    """Single heads, window 1, nothing kept, more kept than the window,
    no window, no rotation, rotation of the whole head, no frequency
    blend, no feed-forward, one group, all groups kept, groups of one,
    all experts chosen, no pair table, no logit cap, unit scales."""
    toks = tokens(24, 7, vocab=31)
    base = {"architecture": "Kazozen", "vocab": 31, "width": 16,
            "norm": {"eps": 1e-6}}
    full = {"embedding": {"scale": 2.0, "bigram": {"buckets": 5,
                                                   "mul_prev": 1,
                                                   "mul_cur": 1}},
            "logit_softcap": 3.0}
    r8 = rot_cfg(8)
    variants = [
        dict(full, layers=[layer(mixer_cfg(1, 1, 8, 8, 1.0, 1, 0, r8),
                                 dense_cfg(8, 100.0))]),
        dict(full, layers=[layer(mixer_cfg(2, 1, 8, 4, 0.5, 3, 9, r8), None),
                           layer(mixer_cfg(2, 1, 8, 4, 0.5, 1, 1, r8,
                                           kv_from=0),
                                 moe_cfg(8, 4, 4, 1, 1, 0.3))]),
        dict(full, layers=[layer(mixer_cfg(2, 2, 6, 6, 0.5, 0, 0, None),
                                 moe_cfg(8, 4, 2, 4, 2, 5.0))]),
        dict(layers=[layer(mixer_cfg(2, 2, 8, 8, 0.5, 5, 2,
                                     rot_cfg(8, scaling=False)),
                           moe_cfg(8, 6, 3, 2, 2, 1.0))]),
        dict({"embedding": {"scale": 1.0}},
             layers=[layer(mixer_cfg(4, 1, 4, 2, 0.7, 100, 0, rot_cfg(2)),
                           moe_cfg(4, 3, 1, 0, 0, 1.0))]),
    ]
    for i, extra in enumerate(variants):
        raw = dict(base, **extra)
        eng, W = make_engine(raw, device, blocks=8, seed=i)
        want = oracle.forward(toks, W, raw)
        got = run_schedule(eng, [[("a", toks[:2], [0, 1])],
                                 [("a", toks[2:19], list(range(17)))],
                                 [("a", toks[19:20], [0])],
                                 [("a", toks[20:], list(range(4)))]])
        rows = torch.stack([got["a"][p] for p in range(len(toks))])
        assert rel_err(rows, want) < TOL, i


def test_config_is_checked():
    raw = small_config()
    raw["layers"][1]["mixer"]["kv_from"] = 1
    with pytest.raises(ValueError):
        registry.model_config_from_dict(raw)
    raw = small_config()
    raw["layers"][3]["mixer"]["kv_from"] = 1     # a borrower, not an owner
    with pytest.raises(ValueError):
        registry.model_config_from_dict(raw)
    raw = small_config()
    raw["layers"][1]["mlp"]["router"]["groups"] = {"count": 4, "keep": 2}
    with pytest.raises(ValueError):
        make_engine(raw, "cpu")
    raw = small_config()
    raw["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        registry.model_config_from_dict(raw)


def _write_checkpoint(tmp_path, raw, W):
    from safetensors.torch import save_file

    d = tmp_path / "model"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(raw))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()},
              str(d / "model.safetensors"))
    return str(d)


def test_checkpoint_directory_roundtrip(tmp_path):
    raw = small_config()
    eng, W = make_engine(raw, "cpu", seed=5)
    path = _write_checkpoint(tmp_path, raw, W)
    mc = registry.get_model_config(path)
    assert mc.architecture == "Kazozen" and mc.model_path == path
    assert registry.required_extensions(mc) == ("seqmix", "moe")
    mc.dtype = "float32"
    cfg = EngineConfig(
        model=mc, cache=CacheConfig(num_gpu_blocks=16,
                                    enable_prefix_caching=False),
        scheduler=SchedulerConfig(max_num_seqs=2, max_num_batched_tokens=256,
                                  max_model_len=256), enforce_eager=True,
        num_state_slots=2)
    eng2 = LLMEngine(cfg, device="cpu")
    Wb = {k: v.to(torch.bfloat16).to(F64) for k, v in W.items()}
    toks = tokens(20, 3)
    got = run_schedule(eng2, [[("a", toks, list(range(20)))]])
    rows = torch.stack([got["a"][p] for p in range(20)])
    assert rel_err(rows, oracle.forward(toks, Wb, raw)) < TOL
    # a checkpoint that lacks a tensor, or holds an unknown one, is refused
    from safetensors.torch import load_file, save_file

    t = load_file(os.path.join(path, "model.safetensors"))
    sink = t.pop("l1.mix.sink")
    save_file(t, os.path.join(path, "model.safetensors"))
    with pytest.raises(ValueError):
        LLMEngine(cfg, device="cpu")
    t["l1.mix.sink"] = sink
    t["l1.mix.k"] = t["l0.mix.k"].clone()   # a borrowing layer has no keys
    save_file(t, os.path.join(path, "model.safetensors"))
    with pytest.raises(ValueError):
        LLMEngine(cfg, device="cpu")


def test_schedule_replay_program(tmp_path):
    """bin/trace_run as a subprocess on a checkpoint directory, with a
    cache pool smaller than the sum of its requests."""
    raw = small_config()
    eng, W = make_engine(raw, "cpu", seed=6)
    path = _write_checkpoint(tmp_path, raw, W)
    Wb = {k: v.to(torch.bfloat16).to(F64) for k, v in W.items()}
    a, b, c = tokens(50, 1), tokens(33, 2), tokens(40, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [29]},
                                {"id": "b", "tokens": b[:2], "want": [0, 1]}],
         "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[30:31], "want": [0]},
                                {"id": "b", "tokens": b[2:], "want": [30]}],
         "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": a[31:], "want": []}],
         "end": ["a"]},
        {"step": 3, "entries": [{"id": "c", "tokens": c, "want": [0, 39]}],
         "end": ["c"]},
    ]
    out = tmp_path / "out"
    p = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model",
         path, "--dtype", "float32", "--out", str(out), "--max-tokens", "96",
         "--device", "cpu"],
        input="\n".join(json.dumps(s) for s in steps) + "\n",
        capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.split("\n") if l.startswith("done")] == [
        "done 0", "done 1", "done 2", "done 3"]
    import numpy as np

    V = raw["vocab"]
    wa, wb, wc = (oracle.forward(t, Wb, raw) for t in (a, b, c))
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", "<f4").reshape(-1, V))
    g1 = torch.from_numpy(np.fromfile(out / "1.f32", "<f4").reshape(-1, V))
    g3 = torch.from_numpy(np.fromfile(out / "3.f32", "<f4").reshape(-1, V))
    assert not (out / "2.f32").exists()
    assert rel_err(g0, torch.stack([wa[29], wb[0], wb[1]])) < TOL
    assert rel_err(g1, torch.stack([wa[30], wb[32]])) < TOL
    assert rel_err(g3, torch.stack([wc[0], wc[39]])) < TOL


def test_bf16_mode_stays_close_to_oracle():
    raw = small_config()
    eng, W = make_engine(raw, "cpu", dtype="bfloat16", seed=2)
    toks = tokens(40, 5)
    want = oracle.forward(toks, W, raw)
    got = run_schedule(eng, [[("a", toks[:17], list(range(17)))],
                             [("a", toks[17:], list(range(23)))]])
    rows = torch.stack([got["a"][p] for p in range(40)])
    d = (rows.double() - want)
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()
    assert err.median() < 0.05


# ------------------------------------------------------------- GPU only

def tiled_config():
    """Head sizes with MFMA tile kernels, expert sizes the MFMA grouped
    GEMM takes, windows shorter than the prompts."""
    r = rot_cfg(32, base=10000.0, factor=2.0, original=128, fast=16.0,
                slow=1.0)
    big = dict(heads=4, kv_heads=2, dim=64, vdim=64, scale=0.125, rot=r)
    return {
        "architecture": "Kazozen", "vocab": 300, "width": 128,
        "norm": {"eps": 1e-5},
        "embedding": {"scale": 4.0, "bigram": {"buckets": 211, "mul_prev": 29,
                                               "mul_cur": 13}},
        "logit_softcap": 12.0,
        "layers": [
            layer(mixer_cfg(window=100, keep=5, **big), dense_cfg(192, 1.5)),
            layer(mixer_cfg(window=70, keep=0, kv_from=0, **big),
                  moe_cfg(64, 8, 2, 4, 3, 2.0)),
            layer(mixer_cfg(heads=2, kv_heads=1, dim=128, vdim=128,
                            scale=0.09, window=300, keep=70,
                            rot=rot_cfg(128, scaling=False)),
                  moe_cfg(64, 4, 1, 2, 1, 1.0)),
        ],
    }


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_engine_matches_oracle_at_tiled_sizes(dtype):
    raw = tiled_config()
    eng, W = make_engine(raw, "cuda", dtype=dtype, blocks=80)
    a, b = tokens(520, 1, 300), tokens(150, 2, 300)
    wa, wb = oracle.forward(a, W, raw), oracle.forward(b, W, raw)
    ask = lambda n, k=16: list(range(0, n, max(n // k, 1)))
    steps = [
        [("a", a[:300], ask(300)), ("b", b[:2], [0, 1])],
        [("a", a[300:430], ask(130)), ("b", b[2:3], [0])],
        [("b", b[3:140], ask(137)), ("a", a[430:431], [0])],
    ]
    steps += [[("a", [x], [0]), ("b", [y], [0])]
              for x, y in zip(a[431:441], b[140:150])]
    steps.append([("a", a[441:], ask(79)), ("end", "a"), ("end", "b")])
    got = run_schedule(eng, steps)
    for rid, want in (("a", wa), ("b", wb)):
        ps = sorted(got[rid])
        rows = torch.stack([got[rid][p] for p in ps])
        d = rows.double() - want[ps]
        d = d - d.mean(-1, keepdim=True)
        w = want[ps] - want[ps].mean(-1, keepdim=True)
        err = d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()
        if dtype == "float32":
            assert err.max() < TOL, rid
        else:
            assert err.median() < 0.05, rid


@pytest.mark.gpu
def test_hipgraph_decode_replays_match_oracle():
    raw = small_config()
    eng, W = make_engine(raw, "cuda", eager=False, blocks=32)
    reqs = [tokens(19, 1), tokens(33, 2), tokens(9, 3)]
    want = [oracle.forward(t, W, raw) for t in reqs]
    steps = [[(f"r{i}", t[:-8], []) for i, t in enumerate(reqs)]]
    for k in range(8, 0, -1):
        steps.append([(f"r{i}", [t[len(t) - k]], [0])
                      for i, t in enumerate(reqs)])
    got = run_schedule(eng, steps)
    for i, t in enumerate(reqs):
        ps = sorted(got[f"r{i}"])
        assert ps == list(range(len(t) - 8, len(t)))
        rows = torch.stack([got[f"r{i}"][p] for p in ps])
        assert rel_err(rows, want[i][ps]) < TOL


@pytest.mark.gpu
def test_generation_with_graph_replay():
    raw = small_config()
    eng, W = make_engine(raw, "cuda", eager=False, max_seqs=2, budget=16,
                         seed=4)
    prompts = [tokens(21, 31), tokens(9, 32), tokens(14, 33)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=10))
    for p, o in zip(prompts, outs):
        assert o.output_token_ids == oracle.greedy(p, W, raw, 10)

#!/usr/bin/env python3
"""FusionInfer-AMD flagship serving benchmark.

Measures the BASELINE.json metric — goodput (completed requests/s) and p50
TTFT for Qwen3-8B serving on MI355X — on synthetic requests with
random-init weights (no network in this environment; BASELINE.md documents
that the reference publishes no numbers of its own).

One rank per GPU (DP replicas, weak scaling — the reference's `replicas`
orchestration). Each rank runs a closed-loop load: target
concurrency is kept topped up; a bench "step" is one engine iteration
(one continuous-batching scheduler step + forward). Timed region:
barrier + torch.cuda.synchronize on both sides of EXACTLY --steps steps.

Measurement stability (round-2): before the timed window the closed loop
is ramped until every initially-admitted request has completed and been
replaced (full turnover), so the window sees steady-state serving only.
Goodput is reported as (generated tokens / elapsed) / E[tokens per
request]; E[tokens/req] == --gen-len exactly by construction of the load
(gen lengths uniform with mean gen_len), so this equals completed
requests / elapsed in expectation but with far lower variance in short
windows (completions are a count of ~1/step; token throughput is stable
per step). The raw completion count and completions/s are also reported.
TTFT samples come only from requests admitted after the turnover ramp
(steady-state admissions), never from the synchronized initial burst.

Usage:
  python bench.py --gpus 1 --steps 64 --warmup 16
  python -m torch.distributed.run --nnodes=1 --nproc-per-node N \
      --master-addr 127.0.0.1 bench.py --gpus N --steps K --warmup W
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import time

import torch
import torch.distributed as dist


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=16)
    p.add_argument("--model", type=str, default="Qwen3-8B")
    p.add_argument("--prompt-len", type=int, default=1024)
    p.add_argument("--gen-len", type=int, default=128)
    p.add_argument("--concurrency", type=int, default=256)
    p.add_argument("--max-batched-tokens", type=int, default=8192)
    p.add_argument("--admission-ms", type=float, default=None,
                   help="admission-hysteresis aging window (scheduler "
                        "default when unset)")
    p.add_argument("--enforce-eager", action="store_true")
    p.add_argument("--kv-cache-dtype", choices=["auto", "fp8"], default="auto",
                   help="fp8 = e4m3 KV cache (halves KV bytes)")
    p.add_argument("--quantization", choices=["fp8"], default=None,
                   help="opt-in fp8 serving mode (headline stays bf16)")
    p.add_argument("--tp", type=int, default=1, help="tensor-parallel degree")
    p.add_argument("--shared-prefix-len", type=int, default=0,
                   help="shared-prefix workload (BASELINE config #4): each "
                        "prompt = one of 8 shared prefixes of this length + "
                        "a unique tail; exercises prefix caching")
    p.add_argument("--spec-tokens", type=int, default=0,
                   help="enable ngram speculative decoding with this draft "
                        "length, and make prompts locally repetitive so the "
                        "prompt-lookup proposer has matches (spec-decode "
                        "workload mode; headline stays spec-off)")
    p.add_argument("--mixer-compare", action="store_true",
                   help="instead of the serving benchmark: prefill and "
                        "decode token throughput of the Kazozen, Momedra, "
                        "Sefalorn and Pinuvik designs at real-model layer "
                        "sizes (random "
                        "weights) next to the Qwen3-style transformer of "
                        "the same sizes")
    p.add_argument("--mc-sizes", default="2048x16,4096x32",
                   help="WIDTHxHEADS list for --mixer-compare (head dim "
                        "128, kv heads = heads/4, ff = 3*width)")
    p.add_argument("--mc-archs",
                   default="kazozen,momedra,sefalorn,pinuvik,transformer")
    p.add_argument("--mc-layers", type=int, default=4)
    p.add_argument("--mc-prompt", type=int, default=2048)
    p.add_argument("--mc-prefill-seqs", type=int, default=4)
    p.add_argument("--mc-decode-batch", type=int, default=64)
    p.add_argument("--mc-chunk", type=int, default=1024,
                   help="attention chunk / window (mask size) of the "
                        "Pinuvik, Sefalorn and Kazozen layers")
    return p.parse_args()


def _mixer_compare_config(arch, width, heads, layers, chunk, vocab=32000):
    from fusioninfer_amd.models.registry import (
        get_model_config,
        model_config_from_dict,
    )

    kv, dim, ff = max(heads // 4, 1), 128, 3 * width
    if arch == "transformer":
        mc = get_model_config("Qwen3-8B")
        mc.name = f"qwen3-style-{width}x{heads}"
        mc.hidden_size, mc.num_layers = width, layers
        mc.num_heads, mc.num_kv_heads, mc.head_dim = heads, kv, dim
        mc.intermediate_size, mc.vocab_size = ff, vocab
        return mc
    if arch == "kazozen":
        # windowed sink attention with 4 kept first keys; every second
        # layer reads the keys and values of the layer before it; dense
        # and routed feed-forwards alternate, the routed ones' active size
        # (top * ff) equals the dense ff
        rot = {"dims": dim, "base": 1e6,
               "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0,
                           "slow": 1.0}}

        def mixer(src=None):
            m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim,
                 "scale": dim ** -0.5, "rot": rot,
                 "mask": {"size": chunk, "keep_first": 4}}
            if src is not None:
                m["kv_from"] = src
            return m

        moe = {"kind": "moe", "expert": {"ff": ff // 2, "limit": 7.0},
               "router": {"experts": 8, "top": 2,
                          "groups": {"count": 4, "keep": 2}}}
        dense = {"kind": "dense", "ff": ff, "limit": 7.0}
        raw = {"architecture": "Kazozen", "vocab": vocab, "width": width,
               "norm": {"eps": 1e-5},
               "embedding": {"scale": 1.0,
                             "bigram": {"buckets": 65521, "mul_prev": 37,
                                        "mul_cur": 19}},
               "logit_softcap": 30.0,
               "layers": [
                   {"type": "attention",
                    "mixer": mixer(i - 1 if i % 2 else None),
                    "mlp": dense if i % 2 == 0 else moe}
                   for i in range(layers)]}
        mc = model_config_from_dict(raw)
        mc.name = f"kazozen-{width}x{heads}"
        return mc
    if arch == "momedra":
        # gated attention, latent attention (run twice as a repeated span)
        # and the gated recurrence in turn; dense and routed feed-forwards
        # alternate, the routed ones' active size (shared + top * ff)
        # equals the dense ff
        moe = {"kind": "moe", "expert": {"ff": ff // 4},
               "router": {"experts": 8, "top": 2},
               "shared": {"ff": ff // 2}}
        dense = {"kind": "dense", "ff": ff}
        attention = {
            "type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim,
                      "vdim": dim, "scale": dim ** -0.5,
                      "q_temp": {"coef": 0.1, "every": 1024}},
            "mlp": dense}
        latent = {
            "type": "latent_attention",
            "mixer": {"heads": heads, "dim": 96, "rot_dim": 32, "vdim": dim,
                      "kv_rank": 256, "scale": dim ** -0.5,
                      "rot": {"base": 1e6, "dims": 32}},
            "mlp": moe}
        rglru = {
            "type": "rglru",
            "mixer": {"width": width, "blocks": heads, "conv": 4},
            "mlp": dense}
        unit = [attention, latent, rglru]
        n_layers = max(layers - 1, 1)
        raw = {"architecture": "Momedra", "vocab": vocab, "width": width,
               "norm": {"eps": 1e-5}, "residual_mult": 0.5,
               "layers": [unit[i % 3] for i in range(n_layers)]}
        if n_layers >= 2:
            raw["loop"] = {"start": 1, "stop": 2, "times": 2}
        mc = model_config_from_dict(raw)
        mc.name = f"momedra-{width}x{heads}"
        return mc
    if arch == "sefalorn":
        # lightning and parallel layers in turn; the experts' active size
        # (top * ff) equals the dense models' ff
        half = max(heads // 2, 1)
        moe = {"kind": "moe", "expert": {"ff": ff // 2},
               "router": {"experts": 8, "top": 2, "scale": 1.0}}
        lightning = {
            "type": "lightning",
            "mixer": {"heads": heads, "dim": dim, "vdim": dim,
                      "decay": [1.0 - 2.0 ** -(3 + 5 * h / max(heads - 1, 1))
                                for h in range(heads)]},
            "mlp": moe}
        parallel = {
            "type": "parallel",
            "mixer": {
                "left": {"heads": heads, "kv_heads": kv, "dim": dim,
                         "vdim": dim, "scale": dim ** -0.5,
                         "mask": {"size": chunk}},
                "left_scale": 0.5,
                "right": {"heads": half, "kv_heads": half, "dim": dim,
                          "vdim": dim, "conv": 4},
                "right_scale": 0.5},
            "mlp": moe}
        raw = {"architecture": "Sefalorn", "vocab": vocab, "width": width,
               "norm": {"eps": 1e-5}, "logit_scale": 1.0,
               "layers": [lightning if i % 2 == 0 else parallel
                          for i in range(layers)]}
        mc = model_config_from_dict(raw)
        mc.name = f"sefalorn-{width}x{heads}"
        return mc
    layer = {
        "type": "parallel",
        "mixer": {
            "left": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim,
                     "scale": dim ** -0.5, "mask": {"size": chunk},
                     "rot": {"dims": dim, "base": 1e6}},
            # the recurrent half at half the attention's head count
            "right": {"heads": max(heads // 2, 1), "dim": dim,
                      "decay_rank": 64},
        },
        "mlp": {"kind": "dense", "ff": ff},
    }
    raw = {"architecture": "Pinuvik", "vocab": vocab, "width": width,
           "norm": {"eps": 1e-5}, "layers": [layer] * layers,
           "loop": {"start": 0, "stop": 0, "times": 1}}
    mc = model_config_from_dict(raw)
    mc.name = f"pinuvik-{width}x{heads}"
    return mc


def run_mixer_compare(args):
    """Prefill: --mc-prefill-seqs prompts of --mc-prompt tokens as ONE
    engine step (forced_step: the engine's own batch path without
    sampling). Decode: --mc-decode-batch sequences at that context, one
    token each per step (hipGraph replay). Tokens/s per arch and size."""
    from fusioninfer_amd.config import (
        CacheConfig,
        EngineConfig,
        SchedulerConfig,
    )
    from fusioninfer_amd.engine.llm_engine import LLMEngine

    use_cuda = torch.cuda.is_available()
    device = "cuda:0" if use_cuda else "cpu"
    P, NS, B = args.mc_prompt, args.mc_prefill_seqs, args.mc_decode_batch
    rows = []
    for size in args.mc_sizes.split(","):
        width, heads = (int(x) for x in size.lower().split("x"))
        for arch in args.mc_archs.split(","):
            mc = _mixer_compare_config(arch, width, heads, args.mc_layers,
                                       args.mc_chunk)
            tokens_cap = B * (P + 64 + args.steps + args.warmup) + NS * P
            cfg = EngineConfig(
                model=mc,
                cache=CacheConfig(num_gpu_blocks=tokens_cap // 16 + B + NS,
                                  enable_prefix_caching=False),
                scheduler=SchedulerConfig(
                    max_num_seqs=B, max_num_batched_tokens=max(NS * P, B * P),
                    max_model_len=P + 64 + args.steps + args.warmup + 16),
                enforce_eager=args.enforce_eager, seed=7,
                num_state_slots=B + NS,
            )
            engine = LLMEngine(cfg, device=device)
            if hasattr(engine.runner.model, "randomize_small_params"):
                engine.runner.model.randomize_small_params(1)
            gen = torch.Generator().manual_seed(5)
            prompt = lambda: torch.randint(
                0, mc.vocab_size, (P,), generator=gen).tolist()
            sync = torch.cuda.synchronize if use_cuda else (lambda: None)

            def prefill_once(tag):
                ids = [f"{tag}-{i}" for i in range(NS)]
                engine.forced_step([(i, prompt(), [P - 1]) for i in ids], ids)

            for w in range(max(args.warmup // 4, 2)):
                prefill_once(f"w{w}")
            sync()
            n_pf = max(args.steps // 8, 3)
            t0 = time.monotonic()
            for w in range(n_pf):
                prefill_once(f"p{w}")
            sync()
            pf_s = (time.monotonic() - t0) / n_pf
            # decode: admit B contexts (in groups so that one step's
            # activations stay modest), then one token each per step
            ids = [f"d{i}" for i in range(B)]
            for a in range(0, B, NS):
                engine.forced_step(
                    [(i, prompt(), []) for i in ids[a:a + NS]])
            step = lambda: engine.forced_step([(i, [1], [0]) for i in ids])
            for _ in range(args.warmup):
                step()
            sync()
            t0 = time.monotonic()
            for _ in range(args.steps):
                step()
            sync()
            dec_s = (time.monotonic() - t0) / args.steps
            engine.forced_step([], ids)
            rows.append({
                "arch": arch, "width": width, "heads": heads,
                "layers": args.mc_layers,
                "prefill_tokens_per_s": round(NS * P / pf_s, 1),
                "prefill_ms": round(pf_s * 1e3, 3),
                "decode_tokens_per_s": round(B / dec_s, 1),
                "decode_ms_per_step": round(dec_s * 1e3, 3),
            })
            del engine
            if use_cuda:
                torch.cuda.empty_cache()
    print(json.dumps({
        "metric": "mixer-compare tokens/s (prefill, decode)",
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "dtype": "bf16", "data": "synthetic",
        "config": {"prompt_len": P, "prefill_seqs": NS, "decode_batch": B,
                   "chunk": args.mc_chunk},
        "rows": rows,
    }))


class ClosedLoopLoad:
    """Keeps `concurrency` requests in flight; tracks completions + TTFT."""

    def __init__(self, engine, prompt_len: int, gen_len: int, concurrency: int,
                 vocab: int, seed: int, shared_prefix_len: int = 0,
                 repetitive: bool = False):
        self.repetitive = repetitive
        self.engine = engine
        self.gen_len = gen_len
        self.prompt_len = prompt_len
        self.concurrency = concurrency
        self.vocab = vocab
        self.rng = torch.Generator().manual_seed(seed)
        self.completion_times = []
        self.first_token_times = {}
        self.ttfts = []
        self.prefixes = []
        if shared_prefix_len > 0:
            self.prefixes = [
                torch.randint(0, vocab, (shared_prefix_len,),
                              generator=self.rng).tolist()
                for _ in range(8)
            ]

    def _new_prompt(self):
        if self.repetitive:
            # period-P repeated random chunk: summarization/extraction-like
            # texts where ngram prompt-lookup actually lands drafts
            period = 32
            chunk = torch.randint(0, self.vocab, (period,),
                                  generator=self.rng).tolist()
            reps = (self.prompt_len + period - 1) // period
            return (chunk * reps)[: self.prompt_len]
        if self.prefixes:
            i = int(torch.randint(0, len(self.prefixes), (1,),
                                  generator=self.rng))
            tail_len = max(self.prompt_len - len(self.prefixes[i]), 8)
            tail = torch.randint(0, self.vocab, (tail_len,),
                                 generator=self.rng).tolist()
            return self.prefixes[i] + tail
        return torch.randint(
            0, self.vocab, (self.prompt_len,), generator=self.rng
        ).tolist()

    def _new_params(self):
        from fusioninfer_amd.engine.sequence import SamplingParams

        # gen lengths uniform in [gen_len/2, 3*gen_len/2] (mean = gen_len):
        # staggers completions so goodput is measurable in short windows
        lo, hi = max(self.gen_len // 2, 1), self.gen_len + self.gen_len // 2
        n = int(torch.randint(lo, hi + 1, (1,), generator=self.rng))
        return SamplingParams(max_tokens=n, temperature=0.0)

    def top_up(self):
        in_flight = self.engine.num_waiting() + self.engine.num_running()
        for _ in range(self.concurrency - in_flight):
            self.engine.add_request(self._new_prompt(), self._new_params())

    def step(self):
        outs = self.engine.step()
        now = time.monotonic()
        for o in outs:
            if o.finished:
                self.completion_times.append(now)
                if o.ttft is not None:
                    self.ttfts.append(o.ttft)
        self.top_up()


def main():
    args = parse_args()
    if args.mixer_compare:
        return run_mixer_compare(args)
    rank = int(os.environ.get("RANK", "0"))
    world = int(os.environ.get("WORLD_SIZE", "1"))
    local_rank = int(os.environ.get("LOCAL_RANK", "0"))
    # Honest n_gpus: --gpus N is a claim that N ranks are running. Refuse
    # to produce a record that says N GPUs while executing on fewer
    # (e.g. `bench.py --gpus 8` launched without torchrun).
    if args.gpus != world:
        raise SystemExit(
            f"bench.py: --gpus {args.gpus} but WORLD_SIZE={world}. "
            f"Launch N>1 via: python -m torch.distributed.run --nnodes=1 "
            f"--nproc-per-node {args.gpus} --master-addr 127.0.0.1 "
            f"bench.py --gpus {args.gpus} ..."
        )
    use_cuda = torch.cuda.is_available()
    device = f"cuda:{local_rank}" if use_cuda else "cpu"
    if use_cuda:
        torch.cuda.set_device(local_rank)

    distributed = world > 1
    if distributed:
        dist.init_process_group(backend="nccl" if use_cuda else "gloo")

    from fusioninfer_amd.config import (
        CacheConfig,
        EngineConfig,
        ParallelConfig,
        SchedulerConfig,
    )
    from fusioninfer_amd.engine.llm_engine import LLMEngine
    from fusioninfer_amd.models.registry import get_model_config

    mc = get_model_config(args.model)
    mc.quantization = args.quantization
    max_len = args.prompt_len + args.gen_len + 64
    cfg = EngineConfig(
        model=mc,
        cache=CacheConfig(
            num_gpu_blocks=None if use_cuda else 4096,
            gpu_memory_utilization=0.85,
            kv_cache_dtype=args.kv_cache_dtype,
        ),
        scheduler=SchedulerConfig(
            max_num_seqs=args.concurrency,
            max_num_batched_tokens=args.max_batched_tokens,
            max_model_len=max_len,
            **({"prefill_admission_ms": (
                None if args.admission_ms < 0 else args.admission_ms)}
               if args.admission_ms is not None else {}),
        ),
        parallel=ParallelConfig(
            tensor_parallel_size=args.tp, rank=rank, world_size=world
        ),
        seed=1234 + rank,
        enforce_eager=args.enforce_eager,
    )
    if args.spec_tokens > 0:
        from fusioninfer_amd.engine.spec_decode import SpeculativeConfig

        cfg.speculative = SpeculativeConfig(
            num_speculative_tokens=args.spec_tokens,
            disable_by_batch_size=0,  # the bench measures spec as asked;
                                      # pick the regime via --concurrency
        )
    # TP: ranks form DP groups of size tp; only group leaders drive load.
    driver_group = None
    if distributed and args.tp > 1:
        driver_ranks = list(range(0, world, args.tp))
        driver_group = dist.new_group(driver_ranks)

    engine = LLMEngine(cfg, device=device)

    if args.tp > 1 and not engine.is_driver:
        engine.worker_loop()   # released by stop_workers() after timing
        _aggregate_and_report(args, rank, world, distributed, device,
                              use_cuda, 0.0, 0, 0, [], is_driver=False)
        if distributed:
            dist.destroy_process_group()
        return

    load = ClosedLoopLoad(
        engine, args.prompt_len, args.gen_len, args.concurrency,
        mc.vocab_size, seed=99 + rank,
        shared_prefix_len=args.shared_prefix_len,
        repetitive=args.spec_tokens > 0,
    )
    load.top_up()

    def barrier_sync():
        if distributed:
            dist.barrier(group=driver_group)
        if use_cuda:
            torch.cuda.synchronize()

    # Load initialization: ramp the closed loop to FULL TURNOVER — every
    # request of the synchronized initial burst has completed and been
    # replaced by steady-state admissions — so the timed window measures
    # steady-state serving for ANY --steps/--warmup. Bounded.
    ramp_limit = 10 * (args.prompt_len // 64 + 2 * args.gen_len) + 800
    ramp_target = args.concurrency + max(args.concurrency // 4, 4)
    ramp = 0
    while len(load.completion_times) < ramp_target and ramp < ramp_limit:
        load.step()
        ramp += 1
    # TTFT samples before this mark belong to (or overlap) the initial
    # burst; only steady-state admissions count from here on.
    steady_ttft_mark = len(load.ttfts)

    for _ in range(args.warmup):
        load.step()

    barrier_sync()
    t0 = time.monotonic()
    completed_before = len(load.completion_times)
    tokens_before = engine.num_generated_tokens
    ttft_mark = len(load.ttfts)
    for _ in range(args.steps):
        load.step()
    barrier_sync()
    elapsed = time.monotonic() - t0

    completed = len(load.completion_times) - completed_before
    gen_tokens = engine.num_generated_tokens - tokens_before
    # Prefer window-local TTFTs; with too few samples (short windows),
    # widen to all steady-state samples — never to the initial burst.
    ttfts = load.ttfts[ttft_mark:]
    if len(ttfts) < 16:
        ttfts = load.ttfts[steady_ttft_mark:]

    engine.stop_workers()
    spec_stats = None
    if args.spec_tokens > 0 and engine.num_spec_draft_tokens:
        spec_stats = {
            "draft_tokens": engine.num_spec_draft_tokens,
            "accepted_tokens": engine.num_spec_accepted_tokens,
            "accept_rate": round(
                engine.num_spec_accepted_tokens
                / max(engine.num_spec_draft_tokens, 1), 3
            ),
        }
    _aggregate_and_report(args, rank, world, distributed, device, use_cuda,
                          elapsed, completed, gen_tokens, ttfts,
                          is_driver=True, spec_stats=spec_stats)
    if distributed:
        dist.destroy_process_group()


def _aggregate_and_report(args, rank, world, distributed, device, use_cuda,
                          elapsed, completed, gen_tokens, ttfts, is_driver,
                          spec_stats=None):
    if distributed:
        dev = device if use_cuda else "cpu"
        t = torch.tensor([elapsed], dtype=torch.float64, device=dev)
        dist.all_reduce(t, op=dist.ReduceOp.MAX)
        elapsed = float(t.item())
        c = torch.tensor([completed, gen_tokens], dtype=torch.float64,
                         device=dev)
        dist.all_reduce(c)
        completed, gen_tokens = float(c[0].item()), float(c[1].item())
        all_ttfts = [None] * world
        dist.all_gather_object(all_ttfts, ttfts)
        ttfts = [x for lst in all_ttfts for x in lst]

    if rank != 0:
        return
    # Low-variance goodput estimator: token throughput / E[tokens per
    # request]; E[tokens/req] == gen_len exactly by construction of the
    # load, so this equals completions/elapsed in expectation (see module
    # docstring). Raw completions/s reported alongside.
    goodput = (
        (gen_tokens / elapsed) / args.gen_len if elapsed > 0 else 0.0
    )
    completed_per_s = completed / elapsed if elapsed > 0 else 0.0
    p50_ttft_ms = (
        statistics.median(ttfts) * 1000.0 if ttfts else float("nan")
    )
    dp = (world // args.tp) if distributed else args.gpus
    result = {
        "metric": f"goodput req/s ({args.model} serving, closed-loop)",
        "value": round(goodput, 3),
        "unit": "req/s",
        "n_gpus": world if distributed else args.gpus,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1000.0, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": (args.quantization or "bf16")
        + ("+kv_fp8" if args.kv_cache_dtype == "fp8" else ""),
        "data": "synthetic",
        "p50_ttft_ms": round(p50_ttft_ms, 1),
        "completed_requests": int(completed),
        "completed_req_per_s": round(completed_per_s, 3),
        **({"spec_decode": spec_stats} if spec_stats else {}),
        "tokens_per_s": round(gen_tokens / elapsed, 1) if elapsed else 0.0,
        "config": {
            "model": args.model,
            "global_batch": args.concurrency * dp,
            "seq_len": args.prompt_len + args.gen_len,
            "prompt_len": args.prompt_len,
            "gen_len": args.gen_len,
            "parallelism": f"dp{dp}"
            + (f"-tp{args.tp}" if args.tp > 1 else ""),
        },
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()

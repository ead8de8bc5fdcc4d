"""Decode and prefill throughput of LFM2-1.2B sizes on one MI355X, with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole batch: every live request gets its next token (the
model's forward from the cache, the head, and greedy choice of the token that is fed back).
The default run: 16 layers of the 1.2B sizes, bfloat16, batch 8, 512-token random prompts,
context 4,096 with 16-token pages.  Prints one JSON line; for more than one GPU it prints
one line that says so and exits with 2 (this engine runs on one GPU).  ``--workload serve`` and
``--workload long`` measure two other workloads and print a line of their own; ``--workload gemm`` times the
products of a 2,048-token prompt one by one, the hand-written kernel beside the vendor library's.

Roofline of the decode step: the bytes it has to read (every weight it uses once, the keys and
values of the live requests, their convolution state) over its time, against 8 TB/s.  Prefill:
2,048 tokens of one prompt; its flops over its time against 2.5 PFLOP/s (bfloat16 dense).
Beside these published peaks the line gives what this machine delivered in the same run
(``peak_measured``, ``frac_measured``): a plain streaming read of 2 GB, and a 4096 x 4096 x 4096
bfloat16 product by the vendor library and by the hand-written kernel, the better of the two.
"""
import argparse
import json
import sys
import time

import torch

HBM_GBPS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


SIZES = {   # hidden, layers, heads, attention layers, block_ff_dim (before the 2/3 adjustment)
    "1.2b": (2048, 16, 32, [2, 5, 8, 10, 12, 14], 12288),
    "350m": (1024, 16, 16, [2, 5, 8, 10, 12, 14], 6656),
    "2.6b": (2048, 30, 32, [2, 6, 10, 14, 18, 21, 24, 27], 10752),
}


def model_config(size: str = "1.2b", max_position: int = 4096):
    from gesso_amd.config import Lfm2Config
    hidden, layers, heads, attn, ff = SIZES[size]
    return Lfm2Config.from_dict({
        "architectures": ["Lfm2ForCausalLM"], "vocab_size": 65536, "hidden_size": hidden, "num_hidden_layers": layers,
        "num_attention_heads": heads, "num_key_value_heads": 8, "full_attn_idxs": attn,
        "conv_L_cache": 3, "conv_bias": False, "block_ff_dim": ff, "block_auto_adjust_ff_dim": True,
        "block_multiple_of": 256, "block_ffn_dim_multiplier": 1.0, "norm_eps": 1e-5, "rope_theta": 1000000.0,
        "tie_word_embeddings": True, "max_position_embeddings": max_position})


def weight_bytes(engine) -> int:
    """Bytes of every weight a decode step reads once (the tied table counts once: it is the head)."""
    seen, n = set(), 0
    m = engine.model
    tensors = [m.head, m.final_norm.weight]
    for b in m.blocks:
        for part in (b.mixer_norm, b.mixer, b.ffn_norm, b.ffn):
            tensors += [v for v in vars(part).values() if isinstance(v, torch.Tensor)]
    for t in tensors:
        if t.data_ptr() not in seen:
            seen.add(t.data_ptr())
            n += t.numel() * t.element_size()
    return n


def step_flops(cfg, tokens: int, attn_pairs: int, rows_out: int) -> float:
    """Multiply-adds x 2 of one step: projections over `tokens`, attention over visible (query, key) pairs."""
    H, F, d = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    nh, nkv = cfg.num_attention_heads, cfg.num_key_value_heads
    n_attn = sum(t == "full_attention" for t in cfg.layer_types)
    n_conv = cfg.num_hidden_layers - n_attn
    per_tok = n_conv * (3 * H * H + H * H) + n_attn * ((nh + 2 * nkv) * d * H + nh * d * H) \
        + cfg.num_hidden_layers * 3 * H * F
    return 2.0 * (per_tok * tokens + n_attn * 2 * nh * d * attn_pairs + rows_out * H * cfg.vocab_size)


def kv_bytes(cfg, engine, lengths) -> int:
    n_attn = sum(t == "full_attention" for t in cfg.layer_types)
    n_conv = cfg.num_hidden_layers - n_attn
    el = 2 if engine.dtype == torch.bfloat16 else 4
    kv = sum(lengths) * n_attn * 2 * cfg.num_key_value_heads * cfg.head_dim * el
    conv = len(lengths) * n_conv * cfg.hidden_size * (cfg.conv_L_cache - 1) * 4 * 2      # read and written
    return kv + conv


def decode_run(engine, cfg, batch: int, prompt_len: int, steps: int, warmup: int, seed: int, temperature: float = 0.0,
               top_p: float = 1.0):
    """Prefill `batch` random prompts, then time `steps` decode steps (greedy, or with `temperature` > 0 every row
    drawing, from its nucleus with `top_p` < 1).  Returns (seconds, mean context)."""
    from gesso_amd.engine.decode import DecodeLoop
    g = torch.Generator().manual_seed(seed)
    rids = [("bench", seed, i) for i in range(batch)]
    first = []
    for rid in rids:
        engine.add_request(rid)
    from gesso_amd import StepEntry
    prompts = [torch.randint(0, cfg.vocab_size, (prompt_len,), generator=g).tolist() for _ in rids]
    at = 0
    while at < batch:                                   # prompts in steps of at most 8,192 tokens
        n = max(1, min(batch - at, 8192 // prompt_len))
        logits = engine.step([StepEntry(r, p, [prompt_len - 1]) for r, p in zip(rids[at:at + n], prompts[at:at + n])])
        first += logits.argmax(1).tolist()
        at += n
    samplers = None
    if temperature > 0:
        from gesso_amd import Sampler
        samplers = [Sampler(temperature, top_p, seed + i) for i in range(batch)]
    loop = DecodeLoop(engine, rids, first, samplers)
    loop.run(warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    loop.run(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    lengths = [engine.length(r) for r in rids]
    mean_ctx = sum(lengths) / batch - steps / 2.0
    loop.close()
    for rid in rids:
        engine.finish_request(rid)
    return dt, mean_ctx


def prefill_run(engine, cfg, tokens: int, reps: int = 5):
    from gesso_amd import StepEntry
    g = torch.Generator().manual_seed(99)
    ids = torch.randint(0, cfg.vocab_size, (tokens,), generator=g).tolist()
    times = []
    warm = 4          # (a recorded step of portions is recorded at its fourth coming)
    for i in range(reps + warm):
        rid = ("prefill", i)
        engine.add_request(rid)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry(rid, ids, [tokens - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        engine.finish_request(rid)
    times = sorted(times[warm:])
    return times[len(times) // 2]


def measured_ceilings(reps: int = 5) -> dict:
    """What the memory system and the matrix cores deliver here: GB/s of a streaming read of 2 GB (cold: the buffer
    is eight times the last-level cache), TFLOP/s of a 4096^3 bfloat16 product (vendor library, and our kernel)."""
    from gesso_amd.kernels import ops
    ops.lib()
    dev = "cuda:0"
    buf = torch.empty(2 * 1024 ** 3, dtype=torch.uint8, device=dev)
    buf.zero_()

    def best(fn):
        fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            times.append(a.elapsed_time(b) * 1e-3)
        return min(times)

    sink = torch.zeros(8192, dtype=torch.int32, device=dev)
    read = max(buf.numel() / best(lambda: ops.stream_read(buf, blocks, contiguous, sink)) / 1e9
               for blocks in (256, 512, 1024, 2048, 4096, 8192) for contiguous in (False, True))
    del buf
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4096, 4096, generator=g).bfloat16().to(dev)
    w = (torch.randn(4096, 4096, generator=g) * 0.02).bfloat16().to(dev)
    flop = 2.0 * 4096 ** 3
    vendor = flop / best(lambda: torch.mm(x, w.t())) / 1e12
    ours = flop / best(lambda: ops.gemm_mfma(x, w)) / 1e12
    return {"read_gbps": round(read, 1), "mfma_tflops_vendor": round(vendor, 1), "mfma_tflops_ours": round(ours, 1)}


def serve_workload(seed: int = 5, record: bool = True, tune: bool = True, budget: int = 4096) -> dict:
    """LFM2-350M sizes: 64 requests at once, prompts of 64 to 2,048 tokens, 32 to 512 new tokens each, prompt
    portions of 512 tokens beside the decodes of the others, at most ``budget`` tokens a step; the scheduler's own loop,
    greedy."""
    from gesso_amd import Session
    from gesso_amd.engine.scheduler import Request
    from gesso_amd.parts import RuntimeOptions
    cfg = model_config("350m")
    g = torch.Generator().manual_seed(seed)
    n = 64
    plen = torch.randint(64, 2049, (n,), generator=g).tolist()
    olen = torch.randint(32, 513, (n,), generator=g).tolist()
    sess = Session(cfg, random_weights_seed=0, context_length=4096, max_num_seqs=64, chunk_size=512,
                   max_num_batched_tokens=budget, max_tokens=n * 2624,
                   kernel_options=RuntimeOptions(record_portions=record, tune_library=tune))
    stamps = {}

    def run():
        sched = sess.scheduler()
        reqs = []
        for i in range(n):
            prompt = torch.randint(0, cfg.vocab_size, (plen[i],), generator=g).tolist()
            stamps[i] = []
            reqs.append(sched.add(Request(("serve", i), prompt, olen[i], None, (), (),
                                          lambda tok, i=i: stamps[i].append(time.perf_counter()))))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while sched.has_work():
            sched.step()
        torch.cuda.synchronize()
        return t0, time.perf_counter(), sched, reqs

    run()                                   # once to record the decode graphs and warm the library
    t0, t1, sched, reqs = run()
    new = sum(len(r.output) for r in reqs)
    ttft = [stamps[i][0] - t0 for i in range(n)]
    tpot = [(stamps[i][-1] - stamps[i][0]) / (len(stamps[i]) - 1) for i in range(n) if len(stamps[i]) > 1]
    return {"metric": "continuous batching, LFM2-350M sizes: new tokens a second over the whole run",
            "value": round(new / (t1 - t0), 1), "unit": "tok/s", "seconds": round(t1 - t0, 3), "requests": n,
            "prompt_tokens": sum(plen), "new_tokens": new, "prompt_tok_s": round(sum(plen) / (t1 - t0), 1),
            "mean_ttft_ms": round(1e3 * sum(ttft) / n, 2), "mean_tpot_ms": round(1e3 * sum(tpot) / len(tpot), 3),
            "steps": sched.stats["steps"], "preemptions": sched.stats["preemptions"], "chunk": 512,
            "token_budget": budget, "recorded_steps": getattr(sess.engine.recorder, "replays", 0), "dtype": "bf16", "data": "synthetic: uniform random token ids, random weights N(0, 0.02)"}


def gemm_workload(reps: int = 10) -> dict:
    """The products of a 2,048-token prompt at LFM2-1.2B sizes, one by one: the hand-written matrix-core kernel (plain,
    and gate|up with its SwiGLU epilogue) beside the vendor library's, microseconds each on random data."""
    from gesso_amd.kernels import ops
    ops.lib()
    dev = "cuda:0"
    g = torch.Generator(device="cpu").manual_seed(3)
    out = {"metric": "products of 2,048 rows at LFM2-1.2B sizes, microseconds (ours plain / ours with SwiGLU / vendor)",
           "unit": "us", "dtype": "bf16", "data": "synthetic: normal activations, weights N(0, 0.02)"}

    def us(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return round((time.perf_counter() - t0) / reps * 1e6, 1)

    for name, (n, k) in {"gate_up": (16384, 2048), "in_proj": (6144, 2048), "down": (2048, 8192),
                         "out_proj": (2048, 2048), "qkv": (3072, 2048)}.items():
        x = torch.randn(2048, k, generator=g).bfloat16().to(dev)
        w = (torch.randn(n, k, generator=g) * 0.02).bfloat16().to(dev)
        row = {"ours": us(lambda: ops.gemm_mfma(x, w)), "vendor": us(lambda: torch.mm(x, w.t()))}
        if name == "gate_up":
            row["ours_swiglu"] = us(lambda: ops.gemm_mfma(x, w, swiglu=True))
            row["vendor_then_swiglu"] = us(lambda: ops.swiglu(torch.mm(x, w.t())))
        out[name] = row
    return out


def stages_workload(batch: int = 8, steps: int = 32) -> dict:
    """The decode step of LFM2-1.2B sizes stage by stage (the decode stage profiler: HIP events around each stage of
    an eagerly launched step; the recorded step itself is faster by what the launches cost)."""
    from gesso_amd import Engine, StepEntry
    cfg = model_config()
    engine = Engine.from_config(cfg, seed=0, dtype="bfloat16", page_size=16, max_context=4096,
                                max_tokens=batch * 1024, num_slots=batch + 1)
    g = torch.Generator().manual_seed(2)
    rids, first = [("st", i) for i in range(batch)], []
    for rid in rids:
        engine.add_request(rid)
        ids = torch.randint(0, cfg.vocab_size, (512,), generator=g).tolist()
        first.append(int(engine.step([StepEntry(rid, ids, [511])]).argmax(1)[0]))
    ids, _ = engine.decode(rids, first, 8)                      # records the graph, warms everything
    prof = engine.profile_decode(True)
    engine.decode(rids, ids[-1].tolist(), 4)                    # eager warm-up of the profiled path
    prof = engine.profile_decode(True)
    engine.decode(rids, ids[-1].tolist(), steps)
    r = prof.report()
    out = {"metric": "decode step of LFM2-1.2B sizes by stage, milliseconds a step (eager launches)", "batch": batch,
           "steps": r["steps"], "step_ms": round(r["step_ms"], 4), "other_ms": round(r["other_ms"], 4)}
    out.update({f"stage_{k}": round(v, 4) for k, v in r["stages_ms"].items()})
    out.update({f"sub_{k}": round(v, 4) for k, v in r["substages_ms"].items()})
    return out


def long_workload(seed: int = 6) -> dict:
    """LFM2-2.6B sizes: prompts of 32,768 tokens in portions of 2,048, then 256 decode steps of 8 such requests."""
    from gesso_amd import Engine, StepEntry
    from gesso_amd.engine.decode import DecodeLoop
    ctx_len, chunk, batch, steps = 32768, 2048, 8, 256
    cfg = model_config("2.6b", max_position=ctx_len + 512)
    from gesso_amd.parts import RuntimeOptions
    engine = Engine.from_config(cfg, seed=0, dtype="bfloat16", page_size=16, max_context=ctx_len + 512,
                                max_tokens=batch * (ctx_len + 512), num_slots=batch + 1,
                                options=RuntimeOptions(tune_library=True))
    g = torch.Generator().manual_seed(seed)
    rids, first, times = [("long", i) for i in range(batch)], [], []
    for rid in rids:
        engine.add_request(rid)
        ids = torch.randint(0, cfg.vocab_size, (ctx_len,), generator=g).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for at in range(0, ctx_len, chunk):
            last = at + chunk >= ctx_len
            logits = engine.step([StepEntry(rid, ids[at:at + chunk], [chunk - 1] if last else [])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        first.append(int(logits.argmax(1)[0]))
    prefill = sorted(times[1:])[len(times[1:]) // 2]            # the first prompt warms the library up
    loop = DecodeLoop(engine, rids, first)
    loop.run(8)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    loop.run(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    wbytes = weight_bytes(engine)
    mean_ctx = ctx_len + 8 + steps / 2.0
    bytes_step = wbytes + kv_bytes(cfg, engine, [mean_ctx] * batch)
    flops = step_flops(cfg, ctx_len, ctx_len * (ctx_len + 1) // 2, 1)
    return {"metric": "LFM2-2.6B sizes at a context of 32,768: decode tok/s at batch 8", "value": round(batch * steps / dt, 1),
            "unit": "tok/s", "ms_per_step": round(dt / steps * 1e3, 4), "decode_gb_per_step": round(bytes_step / 1e9, 3),
            "decode_roofline_frac": round(bytes_step / (dt / steps) / 1e9 / HBM_GBPS, 4),
            "prefill_tok_s": round(ctx_len / prefill, 1), "prefill_s": round(prefill, 4), "prefill_chunk": chunk,
            "prefill_frac": round(flops / prefill / PEAK_FLOPS["bf16"], 4), "layers": cfg.num_hidden_layers,
            "weights_gb": round(wbytes / 1e9, 3), "dtype": "bf16",
            "data": "synthetic: uniform random token ids, random weights N(0, 0.02)"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--size", default="1.2b", choices=sorted(SIZES), help="the layer sizes (the default line: 1.2b)")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--temperature", type=float, default=0.0, help="the main decode run draws at this temperature (0: greedy)")
    ap.add_argument("--top-p", type=float, default=1.0, help="with --temperature: draws from the nucleus of this mass")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points and the prefill")
    ap.add_argument("--only-prefill", action="store_true", help="measure the 2,048-token prefill alone (for profiling)")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the measurement of what the machine delivers")
    ap.add_argument("--no-tune", action="store_true", help="the vendor library's first choice for every product of many "
                    "rows (for profiles: no tuning runs among the kernels)")
    ap.add_argument("--launched-portions", action="store_true", help="launch the steps with prompt portions kernel by kernel instead of "
                    "replaying recordings of them (the prefill of the default line, --workload serve)")
    ap.add_argument("--token-budget", type=int, default=4096, help="--workload serve: the most tokens a step holds")
    ap.add_argument("--workload", default="decode", choices=["decode", "serve", "long", "gemm", "stages"],
                    help="decode: the default line; serve: continuous batching at LFM2-350M sizes; long: LFM2-2.6B "
                         "sizes at a context of 32,768; gemm: the products of a 2,048-token prompt, ours beside the vendor's; "
                         "stages: the decode step stage by stage")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not measured")
        return 2
    if args.workload != "decode":
        if args.workload == "stages":
            print(json.dumps(stages_workload(args.batch, min(args.steps, 32))))
            return 0
        if args.workload == "serve":
            print(json.dumps(serve_workload(record=not args.launched_portions, tune=not args.no_tune, budget=args.token_budget)))
            return 0
        run = {"long": long_workload, "gemm": gemm_workload}[args.workload]
        print(json.dumps(run()))
        return 0

    from gesso_amd import Engine

    cfg = model_config(args.size)
    layers_full = cfg.num_hidden_layers
    model_name = f"LFM2-{args.size.upper()} sizes"
    if args.layers is not None and args.layers < layers_full:
        import dataclasses
        cfg = dataclasses.replace(cfg, num_hidden_layers=args.layers, layer_types=cfg.layer_types[:args.layers])
    prompt_len, context = 512, 4096
    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    max_batch = max(args.batch, 1 if args.no_points else 256)
    from gesso_amd.parts import RuntimeOptions
    engine = Engine.from_config(cfg, seed=0, dtype=dtype, page_size=16, max_context=context,
                                max_tokens=max_batch * (prompt_len + args.steps + args.warmup + 32) + 4096,
                                num_slots=max_batch + 1,
                                options=RuntimeOptions(tune_library=not args.no_tune, record_portions=not args.launched_portions))
    wbytes = weight_bytes(engine)
    if args.only_prefill:
        sec = prefill_run(engine, cfg, 2048)
        print(json.dumps({"prefill_ms": round(sec * 1e3, 3), "tok_s": round(2048 / sec, 1)}))
        return 0

    dt, mean_ctx = decode_run(engine, cfg, args.batch, prompt_len, args.steps, args.warmup, seed=1,
                              temperature=args.temperature, top_p=args.top_p)
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    bytes_step = wbytes + kv_bytes(cfg, engine, [mean_ctx] * args.batch)
    achieved = bytes_step / (ms * 1e-3) / 1e9
    out = {
        "metric": f"decode tok/s at batch {args.batch} ({model_name}, 512-token prompts)", "value": round(value, 1),
        "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: uniform random token ids, random weights N(0, 0.02)",
        "config": {"model": model_name, "layers": cfg.num_hidden_layers, "layers_full": layers_full,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "ff": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "conv_L_cache": cfg.conv_L_cache, "attn_layers": sum(t == "full_attention" for t in cfg.layer_types),
                   "global_batch": args.batch, "prompt_len": prompt_len, "seq_len": context, "page_size": 16,
                   "parallelism": "single GPU", "weights_gb": round(wbytes / 1e9, 3),
                   "recorded_portions": engine.recorder is not None},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
    }
    ceilings = None
    if not args.no_ceilings and args.dtype == "bf16":
        ceilings = measured_ceilings()
        out["roofline"].update(peak_measured=ceilings["read_gbps"], frac_measured=round(achieved / ceilings["read_gbps"], 4))
    if not args.no_points:
        points = {}
        # (256 requests: more than the weight-streaming products take rows; the loop with the many-row products)
        for b, name in ((1, "decode_b1"), (64, "decode_b64"), (256, "decode_b256")):
            steps = min(args.steps, 128)
            dtb, _ = decode_run(engine, cfg, b, prompt_len, steps, min(args.warmup, 8), seed=10 + b)
            points[name] = round(b * steps / dtb, 1)
        # the same batch as the headline with every row drawing: at a temperature, and from a nucleus
        for name, tp in (("decode_b%d_temperature" % args.batch, 1.0), ("decode_b%d_top_p" % args.batch, 0.9)):
            steps = min(args.steps, 128)
            dtb, _ = decode_run(engine, cfg, args.batch, prompt_len, steps, min(args.warmup, 8), seed=30, temperature=0.8, top_p=tp)
            points[name] = round(args.batch * steps / dtb, 1)
        out["points"] = points
        T = 2048
        sec = prefill_run(engine, cfg, T)
        flops = step_flops(cfg, T, T * (T + 1) // 2, 1)
        out["prefill"] = {"value": round(T / sec, 1), "tokens": T, "ms": round(sec * 1e3, 3),
                          "frac": round(flops / sec / PEAK_FLOPS[args.dtype], 4)}
        if ceilings is not None:
            top = max(ceilings["mfma_tflops_vendor"], ceilings["mfma_tflops_ours"])
            out["prefill"].update(peak_measured=top, frac_measured=round(flops / sec / (top * 1e12), 4),
                                  mfma_tflops_vendor=ceilings["mfma_tflops_vendor"],
                                  mfma_tflops_ours=ceilings["mfma_tflops_ours"])
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())

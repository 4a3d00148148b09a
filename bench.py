"""Decode and prefill throughput of the Llama 3 8B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--shape 8b|1b|70b]

Default run: the 8B layer sizes with random bfloat16 weights, a batch of 8
sequences that start from 512-token random prompts; W untimed decode steps, then
exactly K timed ones (a step = one token for every sequence of the batch: model,
greedy sampling on the device and state upkeep, replayed as a HIP graph, tokens read
back by the host every step as generation does).  `value` is decoded tokens a
second.  The same line carries a 2,048-token prefill, the decode step's HBM
roofline, and as `points` decode at batch 1 and 64, prefills of 512 and 8,192 tokens
(tokens a second), decode at batch 8 from prompts of 8,192 and 32,768 tokens (the
pool of the 64 x 8,192-token cache holds them; only the bound of one sequence is raised
for these), and the 1B shape's workload of `--shape 1b` with an engine of its own.  One
JSON line on stdout.

`--dtype float32` runs the true 32-bit path (float32 weights, cache and activations; peaks:
157.3 TFLOP/s, the same 8 TB/s); with the 8B shape that is for a few layers (`--layers 4`).

`--shape 1b`: the Llama 3.2 1B layer sizes, 16 prompts of 64 to 4,096 tokens (uniform, from a
seed) and then K decoding steps, all of it through the generation loop (`GenerationLoop.run`:
prompts in portions of 8,192 rows, captured decoding steps); once with W steps untimed, then timed.
`--shape 70b`: the 70B layer sizes, batch 8 from 1,024-token prompts, with batch 1 and a
2,048-token prefill as points.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_GBPS = 8000.0  # MI355X published peak
BF16_TFLOPS = 2500.0  # dense MFMA bf16
FP32_TFLOPS = 157.3  # dense MFMA fp32

CONFIG_8B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "intermediate_size": 14336,
    "num_hidden_layers": 32, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "vocab_size": 128256, "max_position_embeddings": 8192, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": None, "tie_word_embeddings": False, "torch_dtype": "bfloat16",
    "bos_token_id": 128000, "eos_token_id": 128001,
}


# the other two shapes that the reference's model family names; the default run and the driver use the 8B one
CONFIG_1B = dict(CONFIG_8B, hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, head_dim=64,
                 max_position_embeddings=8192, tie_word_embeddings=True,
                 rope_scaling={"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                               "original_max_position_embeddings": 8192})
CONFIG_70B = dict(CONFIG_8B, hidden_size=8192, intermediate_size=28672, num_hidden_layers=80, num_attention_heads=64)
SHAPES = {"8b": CONFIG_8B, "1b": CONFIG_1B, "70b": CONFIG_70B}


def weight_bytes_per_step(c, element: int = 2) -> float:
    """Every weight a decode step uses, once: the layers' matrices (`element` bytes an entry) and norms
    (always float32), the final norm and the head (of the embedding table only the batch's rows are read)."""
    d, i, hd = c.hidden_size, c.intermediate_size, c.head_dim
    nh, nkv = c.num_attention_heads, c.num_key_value_heads
    per_layer = element * (d * (nh + 2 * nkv) * hd + nh * hd * d + 3 * d * i) + 4 * 2 * d
    return c.num_hidden_layers * per_layer + element * c.vocab_size * d + 4 * d


def kv_bytes_per_token(c, element: int = 2) -> float:
    return 2 * c.num_key_value_heads * c.head_dim * element * c.num_hidden_layers


def prefill_flops(c, t: int) -> float:
    d, i, hd = c.hidden_size, c.intermediate_size, c.head_dim
    nh, nkv = c.num_attention_heads, c.num_key_value_heads
    linear = 2.0 * t * (d * (nh + 2 * nkv) * hd + nh * hd * d + 3 * d * i)
    attention = 2.0 * 2.0 * nh * hd * t * (t + 1) / 2.0  # causal: scores and values
    return c.num_hidden_layers * (linear + attention) + 2.0 * d * c.vocab_size


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the 8B shape has (0 = all 32)")
    ap.add_argument("--batch", type=int, default=0, help="sequences a decoding step (default: 8; 16 for --shape 1b)")
    ap.add_argument("--prompt-len", type=int, default=0,
                    help="prompt tokens (default: 512; 1024 for --shape 70b; the shortest, 64, for --shape 1b)")
    ap.add_argument("--prompt-len-max", type=int, default=0,
                    help="prompts of unequal lengths, uniform in [--prompt-len, this] (0 = all of --prompt-len; "
                         "4096 for --shape 1b)")
    ap.add_argument("--shape", choices=sorted(SHAPES), default="8b", help="layer sizes (the headline run is 8b)")
    ap.add_argument("--no-points", action="store_true", help="skip the prefill and the batch 1 / 64 points")
    ap.add_argument("--prefill-only", action="store_true", help="run the prefill alone, twice (for profiling)")
    ap.add_argument("--profile", action="store_true",
                    help="device time by operation (HIP events around every kernel call): one prefill of "
                         "--prefill-tokens tokens and --steps direct decoding steps at --batch; prints a table and exits")
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="prompt length of --prefill-only (the reported prefill is always of 2,048 tokens)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16",
                    help="float32: the true 32-bit path (use --layers with the larger shapes)")
    ap.add_argument("--context", type=int, default=0,
                    help="tokens a sequence may hold (default: the shape's 8192); for decoding over longer prompts")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    through_loop = args.shape == "1b"  # the workload with unequal prompts runs through the generation loop
    args.batch = args.batch or (16 if args.shape == "1b" else 8)
    args.prompt_len = args.prompt_len or {"8b": 512, "1b": 64, "70b": 1024}[args.shape]
    if args.shape == "1b" and not args.prompt_len_max:
        args.prompt_len_max = 4096

    import torch

    import longbow_quarrel_amd as lq
    from longbow_quarrel_amd.engine import EngineBackend, GenerationLoop, StepEntry

    cfg = dict(SHAPES[args.shape])
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    if args.context:
        cfg["max_position_embeddings"] = args.context
    config = lq.LlamaConfig.from_dict(cfg)
    slot_len = cfg["max_position_embeddings"]
    max_batch = 64 if (args.shape == "8b" and not (args.no_points or args.prefill_only)) else args.batch
    t0 = time.time()
    element = 2 if args.dtype == "bfloat16" else 4
    peak_tflops = BF16_TFLOPS if args.dtype == "bfloat16" else FP32_TFLOPS
    engine = lq.random_engine(config, seed=0, dtype=args.dtype, max_tokens=max_batch * slot_len, max_slots=max_batch)
    torch.cuda.synchronize()
    print(f"[bench] model and cache ready in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(1234)

    def random_prompt(n: int):
        return torch.randint(0, config.vocab_size, (n,), generator=gen).tolist()

    event_ms = {}  # batch size -> milliseconds a step between two events on the engine's stream (the last run of that size)

    def decode_run(batch: int, prompt_len: int, steps: int, warmup: int):
        """tokens a second, ms a step, mean context during the timed steps"""
        # (a point over a longer context than the configuration's: the pool holds it, the bound of one
        # sequence is raised for it)
        engine.max_sequence_tokens = max(engine.max_sequence_tokens, prompt_len + steps + warmup + 2)
        backend = EngineBackend(engine, lq.SamplingParams(temperature=0.0), use_graphs=True)
        slots = [backend.new_sequence(r, [0]) for r in range(batch)]
        lens = [prompt_len] * batch
        if args.prompt_len_max > prompt_len:
            lens = torch.randint(prompt_len, args.prompt_len_max + 1, (batch,), generator=gen).tolist()
        prompts = [random_prompt(n) for n in lens]
        toks = backend.prefill(slots, prompts)  # in portions of at most 8,192 rows a step
        # as the generation loop does, the backend is told before the last step of a run that none follows: it
        # queues no step ahead then, and exactly `steps` steps run between the two synchronisations
        for i in range(warmup):
            backend.expect_more(i + 1 < warmup)
            toks = backend.decode(slots, toks, False)
        torch.cuda.synchronize()
        # the host's clock between two synchronisations is what is reported; a pair of events on the engine's
        # stream around the same steps says how much of it the device itself was busy
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        first.record(engine.stream)
        t = time.perf_counter()
        for i in range(steps):
            backend.expect_more(i + 1 < steps)
            toks = backend.decode(slots, toks, False)
        last.record(engine.stream)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        event_ms[batch] = first.elapsed_time(last) / steps
        ctx_mean = sum(lens) / batch + warmup + (steps + 1) / 2.0
        for s in slots:
            backend.release(s)
        backend.close()
        return batch * steps / dt, dt / steps * 1e3, ctx_mean

    if args.profile:
        from longbow_quarrel_amd.kernels.timed import TimedKernels

        timed = TimedKernels(engine.kernels)
        engine.kernels = timed

        def show(title, wall_ms):
            rows = timed.report()
            total = sum(ms for _, ms in rows.values())
            print(f"[profile] {title}: {wall_ms:.3f} ms on the host's clock, {total:.3f} ms inside event pairs", file=sys.stderr)
            for op, (calls, ms) in rows.items():
                print(f"[profile]   {ms / total * 100:5.1f}%  {calls:5d} calls  {ms / calls * 1e3:9.1f} us  {op}", file=sys.stderr)
            timed.reset()

        n = args.prefill_tokens
        slots = [engine.new_sequence() for _ in range(args.batch)]
        engine.step([StepEntry(slots[0], random_prompt(n), [n - 1])])  # first launches
        engine.release(slots[0])
        slots[0] = engine.new_sequence()
        timed.reset()
        t = time.perf_counter()
        engine.step([StepEntry(slots[0], random_prompt(n), [n - 1])])
        torch.cuda.synchronize()
        show(f"prefill of {n} tokens", (time.perf_counter() - t) * 1e3)
        engine.release(slots[0])
        slots[0] = engine.new_sequence()
        engine.step([StepEntry(s, random_prompt(args.prompt_len), [args.prompt_len - 1]) for s in slots])
        for _ in range(2):
            engine.step([StepEntry(s, [1], [0]) for s in slots])
        timed.reset()
        t = time.perf_counter()
        for _ in range(args.steps):
            engine.step([StepEntry(s, [1], [0]) for s in slots])
        torch.cuda.synchronize()
        show(f"{args.steps} direct decoding steps at batch {args.batch} (no sampling, not captured)",
             (time.perf_counter() - t) * 1e3)
        return 0
    if args.prefill_only:
        n = args.prefill_tokens
        slot = engine.new_sequence()
        engine.step([StepEntry(slot, random_prompt(n), [n - 1])])
        engine.release(slot)
        slot = engine.new_sequence()
        torch.cuda.synchronize()
        t = time.perf_counter()
        engine.step([StepEntry(slot, random_prompt(n), [n - 1])])
        torch.cuda.synchronize()
        print(f"[bench] prefill of {n} tokens: {(time.perf_counter() - t) * 1e3:.2f} ms", file=sys.stderr, flush=True)
        return 0
    def prefill_point(t_tokens: int):
        slot = engine.new_sequence()
        prompt = random_prompt(t_tokens)
        # once untimed (first launches), then three times on fresh slots: the median
        engine.step([StepEntry(slot, prompt, [t_tokens - 1])])
        engine.release(slot)
        times = []
        for _ in range(3):
            slot = engine.new_sequence()
            torch.cuda.synchronize()
            t = time.perf_counter()
            engine.step([StepEntry(slot, prompt, [t_tokens - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            engine.release(slot)
        dt = sorted(times)[1]
        return {"value": round(t_tokens / dt, 1), "tokens": t_tokens, "ms": round(dt * 1e3, 3),
                "frac": round(prefill_flops(config, t_tokens) / dt / (peak_tflops * 1e12), 4)}

    prefill = None
    points = {}
    def loop_run(eng, conf, batch, lo, hi, steps, warmup):
        """`batch` prompts of lengths uniform in [lo, hi], then `steps` decoding steps, as one call of the
        generation loop; the untimed call before it leaves the captured steps behind for the timed one.
        -> tokens a second, ms a step, mean context, the prompts' figures"""
        own = torch.Generator().manual_seed(7)  # the same prompts whatever else this run has drawn before
        lens = torch.randint(lo, hi + 1, (batch,), generator=own).tolist()
        prompts = [torch.randint(0, conf.vocab_size, (n,), generator=own).tolist() for n in lens]
        backend = EngineBackend(eng, lq.SamplingParams(temperature=0.0), use_graphs=True)
        loop = GenerationLoop(backend, max_batch=batch)
        loop.run(prompts, warmup + 1, stop_ids=[])
        torch.cuda.synchronize()
        res = loop.run(prompts, steps + 1, stop_ids=[])  # the first token comes from the prompts' step
        backend.close()
        assert res.decode_steps == steps and res.batches == 1
        flops = sum(prefill_flops(conf, n) for n in lens)
        prompts_line = {"value": round(res.prefill_tokens / res.prefill_seconds, 1), "tokens": res.prefill_tokens,
                        "ms": round(res.prefill_seconds * 1e3, 3),
                        "frac": round(flops / res.prefill_seconds / (peak_tflops * 1e12), 4)}
        return (batch * res.decode_steps / res.decode_seconds, res.decode_seconds / res.decode_steps * 1e3,
                sum(lens) / batch + (steps + 1) / 2.0, prompts_line)

    if through_loop:
        value, ms_step, ctx_mean, prefill = loop_run(engine, config, args.batch, args.prompt_len, args.prompt_len_max,
                                                     args.steps, args.warmup)
    else:
        value, ms_step, ctx_mean = decode_run(args.batch, args.prompt_len, args.steps, args.warmup)
    step_bytes = weight_bytes_per_step(config, element) + args.batch * ctx_mean * kv_bytes_per_token(config, element)
    achieved = step_bytes / (ms_step * 1e-3) / 1e9
    between_events = event_ms.get(args.batch)
    print(f"[bench] decode b{args.batch}: {value:.1f} tok/s, {ms_step:.3f} ms/step" +
          (f" ({between_events:.3f} ms between events on the stream)" if between_events else ""), file=sys.stderr, flush=True)

    if not args.no_points and not through_loop:
        prefill = prefill_point(2048)
        print(f"[bench] prefill: {prefill}", file=sys.stderr, flush=True)
        v1, _, _ = decode_run(1, args.prompt_len, max(16, args.steps // 2), max(4, args.warmup // 2))
        points = {"decode_b1": round(v1, 1)}
        if args.shape == "8b":
            v64, _, _ = decode_run(64, args.prompt_len, max(16, args.steps // 4), max(4, args.warmup // 2))
            points["decode_b64"] = round(v64, 1)
        if args.shape == "8b" and args.dtype == "bfloat16" and not args.layers and not args.context:
            # further prompt lengths and contexts, so that whoever runs the default line times them too
            for n in (512, 8192):
                points[f"prefill_{n}"] = prefill_point(n)["value"]
            for ctx in (8192, 32768):
                if args.batch * (ctx + 64) <= max_batch * slot_len:
                    v, _, _ = decode_run(args.batch, ctx, max(8, args.steps // 4), max(2, args.warmup // 4))
                    points[f"decode_b{args.batch}_ctx{ctx}"] = round(v, 1)
            # the 1B shape's workload (16 prompts of 64 to 4,096 tokens through the generation loop), with an
            # engine of its own beside this one: what `--shape 1b` runs, with half the steps
            small = lq.LlamaConfig.from_dict(dict(CONFIG_1B))
            engine_1b = lq.random_engine(small, seed=0, dtype="bfloat16", max_tokens=16 * 8192, max_slots=16)
            v, ms, ctx, line_1b = loop_run(engine_1b, small, 16, 64, 4096, max(64, args.steps), max(8, args.warmup))
            bytes_1b = weight_bytes_per_step(small) + 16 * ctx * kv_bytes_per_token(small)
            points["decode_1b_b16"] = round(v, 1)
            points["decode_1b_b16_hbm_frac"] = round(bytes_1b / (ms * 1e-3) / 1e9 / HBM_GBPS, 4)
            points["prefill_1b"] = line_1b["value"]
            del engine_1b
        print(f"[bench] points: {points}", file=sys.stderr, flush=True)

    line = {
        "metric": f"decode tok/s (Llama-3 {args.shape.upper()} shape, {'bf16' if element == 2 else 'fp32'}, batch {args.batch}, " + (
            f"prompts of {args.prompt_len} to {args.prompt_len_max} tokens)" if args.prompt_len_max > args.prompt_len
            else f"{args.prompt_len}-token prompts)"),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "ms_per_step_events": round(between_events, 4) if between_events else None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if element == 2 else "fp32", "data": "synthetic: random weights N(0, 0.02) from a seed, uniform random token ids",
        "config": {
            "model": f"llama3-{args.shape}-shape", "layers": config.num_hidden_layers, "layers_full": full_layers,
            "hidden": config.hidden_size, "heads": config.num_attention_heads,
            "kv_heads": config.num_key_value_heads, "head_dim": config.head_dim,
            "intermediate": config.intermediate_size, "vocab": config.vocab_size,
            "rope_theta": config.rope_theta, "rms_eps": config.rms_norm_eps, "tied": config.tie_word_embeddings,
            "rope_scaling": f"{config.rope_scaling.rope_type} x{config.rope_scaling.factor:g}" if config.rope_scaling else "none",
            "global_batch": args.batch, "seq_len": args.prompt_len,
            "seq_len_max": max(args.prompt_len, args.prompt_len_max), "context": slot_len,
            "new_tokens": args.steps + args.warmup, "sampling": "greedy", "parallelism": "single-gpu",
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

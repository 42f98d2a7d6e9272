"""Decode and prefill throughput of the Qwen3-8B shape with random weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]
                    [--shape 8b|0.6b|32b] [--only decode|prefill|generate] [--prompt P]
                    [--with-32b] [--peaks]

Prints one JSON line.  `value` is decoded tokens per second at the given batch after
512-token prompts (one step = one decode step of the whole batch: the model, greedy
sampling, and the tokens fed back).  `prefill` is one prompt of 2,048 tokens;
`roofline` prices the decode step against HBM bandwidth (every weight it uses once,
plus the cache of the live requests); `points` hold decode at batch 1 and 64, and the
headline batch without HIP graphs.
`--only generate` times the generation loop instead: a batch of prompts with lengths
uniform in [64, 2048] that start together, then `--new-tokens` greedy tokens each (the
workload named for the 0.6B shape, with `--shape 0.6b --batch 32 --context 8192`).
`points` also hold the generation workload of the 0.6B shape (the whole loop, its decode
steps timed as steps, its prompt step) and decode at batch 1 and 16 and the prefill of the
32B shape (`--without-32b` leaves those out).  `points` is flat: beside every rate `<name>`
stand `<name>_ms` (a step), `<name>_GB` (what the step has to read, or `_TFLOP`: what it has
to multiply), `<name>_frac` (of the published peak) and `<name>_frac_measured` (of what the
chip at hand gives).  `decode_b8_launches` and `decode_b8_launch_floor_ms`: the kernel launches
of a decode step, and what a graph of as many launches of a kernel that does nothing takes.
Synthetic token ids, seeded random weights N(0, 0.02).  Peaks are the MI355X's published
ones: HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s; `measured_peaks` (and `--peaks` alone) say what
a plain read kernel and a loop of matrix-core products reach on the GPU at hand, and the
roofline and prefill fractions are given against those as well (`frac_measured`).
"""
import argparse
import json
import sys
import time
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))

HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}
PROMPT = 512
PREFILL_TOKENS = 2048
CONTEXT = 4096


# name: (layers, hidden, heads, kv heads, head_dim, intermediate, tied embeddings)
SHAPES = {
    "8b": (36, 4096, 32, 8, 128, 12288, False),
    "0.6b": (28, 1024, 16, 8, 128, 3072, True),
    "32b": (64, 5120, 64, 8, 128, 25600, False),
}


def model_config(shape, layers):
    import edge_infer_amd as ei
    full, hidden, heads, kv_heads, head_dim, inter, tied = SHAPES[shape]
    return ei.Qwen3Config(vocab_size=151936, hidden_size=hidden,
                          num_hidden_layers=layers or full, num_attention_heads=heads,
                          num_key_value_heads=kv_heads, head_dim=head_dim,
                          intermediate_size=inter, max_position_embeddings=40960,
                          bos_token_id=151643, eos_token_id=151645, rms_norm_eps=1e-6,
                          rope_theta=1e6, tie_word_embeddings=tied)


def step_bytes(cfg, cached_tokens, itemsize):
    """Bytes a decode step has to read: layer and head weights once, and the keys and values
    of the `cached_tokens` tokens that its live requests hold together."""
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    Q, KV = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    layer = (Q + 2 * KV) * H + H * Q + 3 * I * H
    weights = itemsize * (cfg.num_hidden_layers * layer + V * H)
    cache = itemsize * 2 * cfg.num_hidden_layers * KV * cached_tokens
    return weights + cache


def prefill_flops(cfg, lengths):
    """Floating-point operations of one prompt step over prompts of these lengths, each
    wanting the logits of its last token."""
    if isinstance(lengths, int):
        lengths = [lengths]
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    Q, KV = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    tokens = sum(lengths)
    layer = 2 * tokens * ((Q + 2 * KV) * H + H * Q + 3 * I * H)
    attention = sum(2 * 2 * cfg.num_attention_heads * cfg.head_dim * n * (n + 1) / 2
                    for n in lengths)
    return cfg.num_hidden_layers * (layer + attention) + len(lengths) * 2 * V * H


def unequal_prompts(cfg, batch, seed=5):
    """Prompts with lengths uniform in [64, 2048], the generation workload's."""
    import random
    import torch
    rng = random.Random(seed)
    lengths = [rng.randint(64, 2048) for _ in range(batch)]
    g = torch.Generator().manual_seed(1)
    return [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lengths]


def synthetic_prompts(cfg, batch, length, seed):
    import torch
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg.vocab_size, (batch, length), generator=g).tolist()


def measure_decode(model, cfg, batch, steps, warmup, prompt=PROMPT, graphs=True, context=CONTEXT,
                   prompts=None):
    """(mean ms per step, mean context of a sequence during the timed steps, median ms per
    step).  `prompts`: the batch's prompts (of unequal lengths, say) instead of `batch`
    synthetic ones of `prompt` tokens; the mean context is then the mean over them."""
    import torch
    import edge_infer_amd as ei
    from edge_infer_amd.sampling import Sampler, SamplingParams
    session = ei.Session(model, max_tokens=batch * context, max_seqs=batch,
                         max_seq_tokens=context, graphs=graphs)
    sampler = Sampler(model.device)
    greedy = SamplingParams(temperature=0.0)
    if prompts is None:
        prompts = synthetic_prompts(cfg, batch, prompt, seed=100 + batch)
    prompt = sum(len(p) for p in prompts) / len(prompts)
    slots = [session.begin() for _ in range(batch)]
    logits = session.step([(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)], copy=False)
    tokens = sampler(logits, greedy, [], [])
    stamps = []

    def run(count):
        nonlocal tokens
        for _ in range(count):
            logits = session.step([(s, [t], [0]) for s, t in zip(slots, tokens)], copy=False)
            tokens = sampler(logits, greedy, [], [])     # (fetches the tokens: the step is over)
            stamps.append(time.perf_counter())

    run(warmup)
    torch.cuda.synchronize()
    stamps.clear()
    started = time.perf_counter()
    run(steps)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    each = sorted(b - a for a, b in zip([started] + stamps[:-1], stamps))
    median = each[len(each) // 2] if len(each) % 2 else (each[len(each) // 2 - 1] + each[len(each) // 2]) / 2
    mean_context = prompt + warmup + (steps + 1) / 2
    for s in slots:
        session.end(s)
    del session
    torch.cuda.empty_cache()
    return 1000.0 * elapsed / steps, mean_context, 1000.0 * median


def measure_prefill(model, cfg, repeats=3, tokens=PREFILL_TOKENS):
    import torch
    import edge_infer_amd as ei
    session = ei.Session(model, max_tokens=tokens, max_seqs=1)
    prompt = synthetic_prompts(cfg, 1, tokens, seed=7)[0]
    best = None
    for _ in range(repeats + 1):
        slot = session.begin()
        torch.cuda.synchronize()
        started = time.perf_counter()
        session.step([(slot, prompt, [tokens - 1])], copy=False)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        session.end(slot)
        best = elapsed if best is None else min(best, elapsed)
    del session
    torch.cuda.empty_cache()
    return 1000.0 * best


def measure_generate(model, cfg, batch, context, new_tokens, repeats=2):
    """Best wall time of `Session.generate_batch` over a batch of unequal prompts, and the
    time of its prompt step alone."""
    import torch
    import edge_infer_amd as ei
    prompts = unequal_prompts(cfg, batch)
    lengths = [len(p) for p in prompts]
    session = ei.Session(model, max_tokens=batch * context, max_seqs=batch,
                         max_seq_tokens=context)
    total = None
    for _ in range(repeats + 1):
        torch.cuda.synchronize()
        started = time.perf_counter()
        out = session.generate_batch(prompts, max_new_tokens=new_tokens, temperature=0.0,
                                     stop_ids=())
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - started
        total = elapsed if total is None else min(total, elapsed)
    slots = [session.begin() for _ in range(batch)]
    torch.cuda.synchronize()
    started = time.perf_counter()
    session.step([(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)], copy=False)
    torch.cuda.synchronize()
    prompt_s = time.perf_counter() - started
    for s in slots:
        session.end(s)
    del session
    torch.cuda.empty_cache()
    return total, prompt_s, lengths, sum(len(o) for o in out)


def measure_peaks():
    """What a plain read kernel streams (GB/s) and a loop of matrix-core products computes
    (TFLOP/s, bfloat16) on this GPU: the best of a few runs each."""
    import torch
    from edge_infer_amd.csrc import lib
    device = torch.device("cuda")
    data = torch.empty(4 * 1024 ** 3, dtype=torch.uint8, device=device)
    data.fill_(1)
    sink = torch.zeros(4, dtype=torch.int32, device=device)
    fsink = torch.zeros(4, dtype=torch.float32, device=device)

    def best(launch, repeats=5):
        times = []
        for _ in range(repeats + 1):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            launch()
            end.record()
            end.synchronize()
            times.append(begin.elapsed_time(end) * 1e-3)
        return min(times[1:])
    read_s = min(best(lambda: lib.stream_read(data, sink, blocks)) for blocks in (2048, 4096, 8192))
    iters, blocks = 20000, 256 * 8
    mfma_s = min(best(lambda: lib.mfma_loop(iters, blocks, fsink, wide)) for wide in (False, True))
    flops = lib.MFMA_LOOP_FLOPS * iters * blocks * 4
    del data
    torch.cuda.empty_cache()
    return {"hbm_read_GBs": round(data_bytes_of(4) / read_s / 1e9, 1),
            "mfma_bf16_TFLOPs": round(flops / mfma_s / 1e12, 1)}


def measure_launch_floor(model, cfg, batch, replays=50):
    """(kernel launches of one decode step, ms a replay of a graph of as many launches of a
    kernel that does nothing): what the chain of dependent launches alone costs, the floor
    under a step of this design whatever its kernels do."""
    import torch
    import edge_infer_amd as ei
    from edge_infer_amd.csrc import lib
    session = ei.Session(model, max_tokens=batch * 1024, max_seqs=batch, max_seq_tokens=1024,
                         graphs=False)
    prompts = synthetic_prompts(cfg, batch, 64, seed=9)
    slots = [session.begin() for _ in range(batch)]
    session.step([(s, p, [63]) for s, p in zip(slots, prompts)], copy=False)
    before = lib.launches
    session.step([(s, [1], [0]) for s in slots], copy=False)
    count = lib.launches - before
    del session
    lib.empty_launches(4)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        lib.empty_launches(count)
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    started = time.perf_counter()
    for _ in range(replays):
        graph.replay()
    torch.cuda.synchronize()
    return count, 1000.0 * (time.perf_counter() - started) / replays


def data_bytes_of(gib):
    return gib * 1024 ** 3


def decode_point(points, name, cfg, batch, ms, cached_tokens, itemsize, peaks):
    """A decode measurement as flat entries of `points`: tokens a second, a step's time, what
    it has to read, and the fractions of the published and of the measured read rate."""
    nbytes = step_bytes(cfg, cached_tokens, itemsize)
    rate = nbytes / (ms * 1e-3) / 1e9
    points[name] = round(batch * 1000.0 / ms, 1)
    points[name + "_ms"] = round(ms, 4)
    points[name + "_GB"] = round(nbytes / 1e9, 3)
    points[name + "_frac"] = round(rate / HBM_PEAK_GBS, 4)
    points[name + "_frac_measured"] = round(rate / peaks["hbm_read_GBs"], 4)


def prefill_point(points, name, cfg, lengths, ms, dtype, peaks):
    """A prompt step the same way: tokens a second, its time, its operations, fractions of the
    published and of the measured matrix-core rate."""
    flops = prefill_flops(cfg, lengths)
    tokens = lengths if isinstance(lengths, int) else sum(lengths)
    points[name] = round(tokens * 1000.0 / ms, 1)
    points[name + "_ms"] = round(ms, 3)
    points[name + "_TFLOP"] = round(flops / 1e12, 3)
    points[name + "_frac"] = round(flops / (ms * 1e-3) / (PEAK_TFLOPS[dtype] * 1e12), 4)
    if dtype == "bfloat16":
        points[name + "_frac_measured"] = round(flops / (ms * 1e-3)
                                                / (peaks["mfma_bf16_TFLOPs"] * 1e12), 4)


def other_shape_points(args, itemsize, peaks):
    """Decode and prefill figures of the other shapes, as flat numbers for `points`."""
    import torch
    import edge_infer_amd as ei
    points = {}
    cfg = model_config("0.6b", 0)
    model = ei.random_model(cfg, seed=3, dtype=args.dtype)
    batch, new_tokens = 32, 256
    total, prompt_s, lengths, new = measure_generate(model, cfg, batch, 8192, new_tokens, repeats=1)
    points["gen_0.6b_b32_new_tokens_per_s"] = round(new / total, 1)
    points["gen_0.6b_b32_total_ms"] = round(1e3 * total, 1)
    prefill_point(points, "gen_0.6b_b32_prompt_tokens_per_s", cfg, lengths, 1e3 * prompt_s,
                  args.dtype, peaks)
    # the loop's decode steps, timed as steps: the same prompts, then 255 tokens each, all but
    # the first four timed (the mean holds the steps that capture a graph for a new context
    # bound, as the loop's own time does; the median does not)
    ms, context, median = measure_decode(model, cfg, batch, new_tokens - 5, 4, context=8192,
                                         prompts=unequal_prompts(cfg, batch))
    decode_point(points, "gen_0.6b_b32_decode", cfg, batch, ms, batch * context, itemsize, peaks)
    points["gen_0.6b_b32_decode_ms_median"] = round(median, 4)
    del model
    torch.cuda.empty_cache()
    if not args.without_32b:
        cfg = model_config("32b", 0)
        model = ei.random_model(cfg, seed=4, dtype=args.dtype)
        for batch in (1, 16):
            ms, context, _ = measure_decode(model, cfg, batch, 16, 4)
            decode_point(points, f"32b_decode_b{batch}", cfg, batch, ms, batch * context,
                         itemsize, peaks)
        ms = measure_prefill(model, cfg, repeats=2)
        prefill_point(points, "32b_prefill_tokens_per_s", cfg, PREFILL_TOKENS, ms, args.dtype, peaks)
        del model
        torch.cuda.empty_cache()
    return points


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--shape", choices=sorted(SHAPES), default="8b",
                        help="layer sizes: Qwen3-8B (the default and the headline), 0.6B or 32B")
    parser.add_argument("--layers", type=int, default=0,
                        help="layers of the model (0: as many as the shape has)")
    parser.add_argument("--prompt", type=int, default=PROMPT,
                        help="prompt length before the timed decode steps (with --only decode)")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--skip-points", action="store_true")
    parser.add_argument("--only", choices=["decode", "prefill", "generate"], default=None,
                        help="run one workload only and print its figures (for profiling)")
    parser.add_argument("--context", type=int, default=CONTEXT,
                        help="tokens a sequence may hold (with --only generate)")
    parser.add_argument("--new-tokens", type=int, default=256,
                        help="tokens generated for each prompt (with --only generate)")
    parser.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                        help="with --only prefill: the length of the one prompt (the record's "
                             "prefill is always of 2,048 tokens)")
    parser.add_argument("--with-32b", action="store_true", help="(the default; kept for old command lines)")
    parser.add_argument("--without-32b", action="store_true",
                        help="leave the 32B shape (decode at batch 1 and 16, prefill) out of `points`")
    parser.add_argument("--peaks", action="store_true",
                        help="measure the read and matrix-core yardsticks only")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    import edge_infer_amd as ei
    if args.peaks:
        print(json.dumps({"only": "peaks", **measure_peaks(),
                          "published": {"hbm_GBs": HBM_PEAK_GBS, "mfma_bf16_TFLOPs": PEAK_TFLOPS["bfloat16"]}}))
        return 0
    cfg = model_config(args.shape, args.layers)
    full_layers = SHAPES[args.shape][0]
    model = ei.random_model(cfg, seed=2, dtype=args.dtype)
    torch.cuda.synchronize()
    itemsize = 2 if args.dtype == "bfloat16" else 4

    if args.only == "decode":
        ms_step, context, median = measure_decode(model, cfg, args.batch, args.steps, args.warmup,
                                                  args.prompt, context=max(CONTEXT, args.context))
        rate = step_bytes(cfg, args.batch * context, itemsize) / (ms_step * 1e-3) / 1e9
        print(json.dumps({"only": "decode", "shape": args.shape, "batch": args.batch,
                          "ms_per_step": round(ms_step, 4), "ms_per_step_median": round(median, 4),
                          "tokens_per_s": round(args.batch * 1000.0 / ms_step, 1),
                          "context": round(context), "GB/s": round(rate, 1)}))
        return 0
    if args.only == "generate":
        total, prompt_s, lengths, new = measure_generate(model, cfg, args.batch,
                                                         args.context, args.new_tokens)
        prompt_tokens = sum(lengths)
        steps = args.new_tokens - 1          # the first token comes from the prompt step
        print(json.dumps({"only": "generate", "shape": args.shape, "batch": args.batch,
                          "prompt_tokens": prompt_tokens, "new_tokens": new,
                          "total_ms": round(1e3 * total, 1),
                          "new_tokens_per_s": round(new / total, 1),
                          "prompt_step_ms": round(1e3 * prompt_s, 1),
                          "prompt_tokens_per_s": round(prompt_tokens / prompt_s, 1),
                          "ms_per_decode_step": round(1e3 * (total - prompt_s) / max(1, steps), 4)}))
        return 0
    if args.only == "prefill":
        tokens = args.prefill_tokens
        prefill_ms = measure_prefill(model, cfg, tokens=tokens)
        flops = prefill_flops(cfg, tokens)
        print(json.dumps({"only": "prefill", "shape": args.shape, "tokens": tokens,
                          "ms": round(prefill_ms, 3),
                          "TFLOP/s": round(flops / (prefill_ms * 1e-3) / 1e12, 1)}))
        return 0
    ms_step, context, median_step = measure_decode(model, cfg, args.batch, args.steps, args.warmup)
    value = args.batch * 1000.0 / ms_step
    achieved = step_bytes(cfg, args.batch * context, itemsize) / (ms_step * 1e-3) / 1e9
    prefill_ms = measure_prefill(model, cfg)
    flops = prefill_flops(cfg, PREFILL_TOKENS)
    peaks = measure_peaks()
    points = {}
    if not args.skip_points:
        for name, batch in (("decode_b1", 1), ("decode_b64", 64)):
            ms, at, _ = measure_decode(model, cfg, batch, max(8, args.steps // 2), args.warmup)
            decode_point(points, name, cfg, batch, ms, batch * at, itemsize, peaks)
        # the headline batch with every kernel launched by the host instead of from a HIP graph
        ms, at, _ = measure_decode(model, cfg, args.batch, max(8, args.steps // 2), args.warmup,
                                   graphs=False)
        decode_point(points, f"decode_b{args.batch}_eager", cfg, args.batch, ms, args.batch * at,
                     itemsize, peaks)
        # what the step's chain of launches costs with kernels that do nothing
        count, floor_ms = measure_launch_floor(model, cfg, args.batch)
        points[f"decode_b{args.batch}_launches"] = count
        points[f"decode_b{args.batch}_launch_floor_ms"] = round(floor_ms, 4)
    if not args.skip_points and args.shape == "8b":
        del model
        torch.cuda.empty_cache()
        points.update(other_shape_points(args, itemsize, peaks))
    from edge_infer_amd.csrc import lib
    record = {
        "metric": f"decode tokens/s, Qwen3-{args.shape.upper()} shape, batch {args.batch} after "
                  f"{PROMPT}-token prompts",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "ms_per_step_median": round(median_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic token ids, seeded random weights N(0, 0.02)",
        "config": {
            "model": f"Qwen3-{args.shape.upper()} shape", "layers": cfg.num_hidden_layers,
            "layers_full_model": full_layers,
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps,
            "tie_word_embeddings": cfg.tie_word_embeddings, "global_batch": args.batch, "prompt_len": PROMPT,
            "context_capacity": CONTEXT, "seq_len": round(context), "parallelism": "single GPU",
            "kernels": "+".join(lib.loaded_libraries()),
        },
        "prefill": {"value": round(PREFILL_TOKENS * 1000.0 / prefill_ms, 1),
                    "tokens": PREFILL_TOKENS, "ms": round(prefill_ms, 3),
                    "frac": round(flops / (prefill_ms * 1e-3) / (PEAK_TFLOPS[args.dtype] * 1e12), 4),
                    "frac_measured": round(flops / (prefill_ms * 1e-3)
                                           / (peaks["mfma_bf16_TFLOPs"] * 1e12), 4)
                    if args.dtype == "bfloat16" else None},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "frac_measured": round(achieved / peaks["hbm_read_GBs"], 4)},
        "measured_peaks": peaks,
        "points": points,
    }
    print(json.dumps(record))
    return 0


if __name__ == "__main__":
    sys.exit(main())

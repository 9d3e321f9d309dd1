"""The headline measurement: decode tokens per second of a Llama-3-8B-shaped model with
random bfloat16 weights on one MI355X, batch 8 after 1,024-token prompts, beside the
prefill rate at 2,048 tokens, decode at batch 1 and 64, and how far the decode step is
from the memory roofline.  The metric follows the reference's definitions (throughput =
batch x tokens / time, TBT = mean time of a decode step: yalis/engine.py:531-557).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L]

A step is one decode step through the engine's own path: page reservation, the step
function over the paged cache, greedy sampling.  As in ``LLMEngine.generate``, steps that need
no decision of the scheduler are launched one behind the other, each feeding on the tokens the
step before left on the device; the tokens of all timed steps are on the host when the clock
stops.

Beside the headline the one JSON line holds: ``roofline`` (the bytes a decode step has to
read, every weight once and the cache of the live requests, over its time, against 8 TB/s);
``prefill`` (2,048 tokens, the mean of three timed runs, with its fraction of 2.5 PFLOP/s);
``points``: decode at batch 1 and 64 with the same roofline fraction each; TTFT and TBT of the
same workload as ``LLMEngine.generate`` itself reports them; prefill of 512 and 8,192 tokens,
decode at batch 8 behind 8,000-token prompts and at batch 64 behind 4,000-token ones; mixed
steps at the Llama-3.2-3B shape (32 decode streams beside 480-, 992- and 2,016-token portions
of 4,096-token prompts) with their bound max(bytes / 8 TB/s, flops / 2.5 PFLOP/s); decode at
batch 1 / 8 / 64 behind 2,048-token prompts at the Llama-3.1-70B shape (``--no-70b`` leaves
it out); ``breakdown``: the time of a
decode step and of the prefill by kind of work (products, attention, output head, norms),
each with the fraction of the peak that bounds it.
"""
import argparse
import json
import sys
import time

HBM_GBPS = 8000.0  # MI355X published peaks
BF16_FLOPS = 2.5e15

from yalis_amd.models.presets import SHAPES  # name -> (label, config.json dictionary)


def machine_probe(cfg: dict) -> int:
    """What the card gives a kernel that does nothing but read, at the sizes of the shape's
    weight matrices, and a kernel that does nothing but issue bfloat16 matrix-core
    instructions.  The decode products stream their weights once, so the first is their
    practical bound; the second is the bound of any bfloat16 product."""
    import torch

    from yalis_amd.ops.hip import HipOps

    ops = HipOps("cuda:0")
    c, h, g, d = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    inter, vocab = cfg["intermediate_size"], cfg["vocab_size"]
    sizes = {
        "o_proj": h * d * c * 2,
        "qkv_proj": (h + 2 * g) * d * c * 2,
        "down_proj": c * inter * 2,
        "gate_up_proj": 2 * inter * c * 2,
        "head": vocab * c * 2,
    }
    arena = torch.empty(6 << 30, dtype=torch.uint8, device="cuda")
    arena.view(torch.int32).random_(0, 1 << 20)  # small positive floats: no NaN, nothing cached from a memset
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    out = {}
    print("streaming read of one weight matrix (a fresh piece of a 6 GiB arena each time, mean of 20):")
    for name, nbytes in sizes.items():
        best = None
        for wgs, nt in ((512, False), (2048, False), (16384, False), (512, True), (2048, True), (16384, True)):
            offset, total = 0, 0.0
            for rep in range(23):
                if offset + nbytes > arena.numel():
                    offset = 0
                piece = arena[offset : offset + nbytes]
                offset += -(-nbytes // 4096) * 4096
                start.record()
                ops.probe_stream_read(piece, wgs, sink, nontemporal=nt)
                stop.record()
                stop.synchronize()
                if rep >= 3:
                    total += start.elapsed_time(stop)
            us = total / 20 * 1e3
            if best is None or us < best[0]:
                best = (us, wgs, nt)
        tbs = nbytes / (best[0] * 1e-6) / 1e12
        out[name] = {"MB": round(nbytes / 1e6, 1), "us": round(best[0], 1), "TB/s": round(tbs, 2), "workgroups": best[1], "nontemporal": best[2]}
        print(f"  {name:13s} {nbytes / 1e6:8.1f} MB  {best[0]:7.1f} us  {tbs:5.2f} TB/s  ({best[1]} workgroups{', nontemporal loads' if best[2] else ''})")
    wgs, iters = 256 * 8, 20000
    for rep in range(3):
        start.record()
        flops = ops.probe_mfma_bf16(wgs, iters, sink)
        stop.record()
        stop.synchronize()
    pf = flops / (start.elapsed_time(stop) * 1e-3) / 1e15
    print(f"bfloat16 matrix-core loop from registers ({wgs} workgroups of 4 waves, 4 accumulators each): {pf:.2f} PFLOP/s")
    print(json.dumps({"probe": "machine", "stream_read": out, "mfma_bf16_pflops": round(pf, 3)}))
    return 0


def sampling_times(vocab: int, batch: int) -> int:
    """Times the choice of a token alone (no model) at this vocabulary for ``batch`` rows:
    greedy and each sampling rule, on a nearly flat row (what random weights give) and on a
    peaked one (a few dozen likely tokens, as a trained model gives)."""
    import torch

    from yalis_amd.ops.hip import HipOps

    ops = HipOps("cuda:0")
    gen = torch.Generator(device="cuda").manual_seed(0)
    flat = torch.randn(batch, vocab, device="cuda", generator=gen) * 0.3
    peaked = torch.randn(batch, vocab, device="cuda", generator=gen) * 2.5
    peaked[:, :50] += 12.0
    full = lambda v, dt: torch.full((batch,), v, dtype=dt, device="cuda")
    seeds, draws = torch.arange(batch, dtype=torch.int32, device="cuda"), full(0, torch.int32)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    out = {}
    for rows_name, logits in (("flat", flat), ("peaked", peaked)):
        for name, (t, k, p) in (("greedy", (0.0, 0, 1.0)), ("temperature", (1.0, 0, 1.0)), ("top_p 0.8", (1.0, 0, 0.8)),
                                ("top_k 50", (1.0, 50, 1.0)), ("top_k 50, top_p 0.8, T 0.7", (0.7, 50, 0.8))):
            temperature, top_k, top_p = full(t, torch.float32), full(k, torch.int32), full(p, torch.float32)
            run = (lambda: ops.argmax(logits)) if t == 0.0 else (lambda: ops.sample(logits, temperature, top_k, top_p, seeds, draws))
            for _ in range(3):
                run()
            start.record()
            for _ in range(20):
                run()
            stop.record()
            stop.synchronize()
            us = start.elapsed_time(stop) / 20 * 1e3
            out[f"{rows_name}: {name}"] = round(us, 1)
            print(f"  {rows_name:7s} {name:28s} {us:7.1f} us")
    print(json.dumps({"probe": "sampling", "vocab": vocab, "rows": batch, "us": out}))
    return 0


class Shape:
    """The sizes of a configuration that the byte and flop counts need."""

    def __init__(self, cfg: dict):
        self.c, self.h, self.g, self.d = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
        self.inter, self.vocab, self.layers = cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
        self.layer_params = self.c * (self.h + 2 * self.g) * self.d + self.h * self.d * self.c + 3 * self.c * self.inter
        # every weight a decode step reads once: the layers, the norms, the output head (the
        # embedding table itself when tied; of a separate table only a row per token is read)
        self.weight_bytes = 2 * (self.layers * (self.layer_params + 2 * self.c) + self.c + self.vocab * self.c)
        self.kv_bytes_per_token = self.layers * 2 * self.g * self.d * 2

    def decode_bytes(self, batch: int, mean_ctx_tokens: float) -> float:
        """What a decode step has to read: every weight once, the cache of the live requests."""
        return self.weight_bytes + batch * self.c * 2 + mean_ctx_tokens * self.kv_bytes_per_token

    def prefill_flops(self, t: int) -> float:
        return self.layers * (2 * t * self.layer_params + 2 * self.h * self.d * t * t) + 2 * self.vocab * self.c


def make_engine(cfg: dict, max_batch: int, ctx_cap: int, graphs: bool = True, page: int = 64, pool_tokens: int = 0):
    """The engine as a user builds it over random weights of a shape (``LLMEngine.from_random``):
    its runner is what the step-level measurements drive, its ``generate`` what the
    generate-level ones call.  ``pool_tokens``: the pool's size when it is not ``max_batch``
    requests of ``ctx_cap`` tokens."""
    from yalis_amd import InferenceConfig, LLMEngine
    from yalis_amd.config.runtime import EngineConfig

    pages_per_req = -(-ctx_cap // page)
    max_len = min(cfg["max_position_embeddings"], pages_per_req * page)
    engine = EngineConfig(
        page_size=page, num_pages=-(-pool_tokens // page) if pool_tokens else pages_per_req * max_batch, max_num_seqs=max_batch,
        max_model_len=max_len, max_num_batched_tokens=8192, dtype="bfloat16", decode_graphs=graphs,
    )
    ic = InferenceConfig(max_batch_size=max_batch, max_length_of_generated_sequences=max_len, temperature=0.0)
    return LLMEngine.from_random(cfg, ic, precision="bf16", seed=0, engine_config=engine)


def make_runner(cfg: dict, max_batch: int, ctx_cap: int, graphs: bool = True, page: int = 64):
    return make_engine(cfg, max_batch, ctx_cap, graphs, page).runner


def generate_metrics(engine, vocab: int, gen, batch: int, prompt_len: int, n_tokens: int):
    """TTFT and TBT as ``LLMEngine.generate`` itself reports them (the reference's definitions,
    yalis/engine.py:531-557) for ``batch`` prompts of ``prompt_len`` tokens; the second of two
    calls (the first captures the decode graphs)."""
    import torch

    prompts = [torch.randint(0, vocab, (prompt_len,), generator=gen).tolist() for _ in range(batch)]
    metrics = None
    for _ in range(2):
        _, metrics = engine.generate(prompts, tokens_to_generate=n_tokens, ignore_eos=True)
    return metrics


def decode_run(runner, vocab: int, gen, batch: int, prompt_len: int, steps: int, warmup: int):
    """Prefill ``batch`` prompts, then time ``steps`` decode steps launched one behind the other.
    Returns (seconds, mean cached tokens read per step)."""
    import torch

    from yalis_amd.engine.step import StepEntry

    ops = runner.rt.ops
    toks = []
    for r in range(batch):
        assert runner.admit(r)
        prompt = torch.randint(0, vocab, (prompt_len,), generator=gen).tolist()
        assert runner.reserve(r, len(prompt))
        toks.append(ops.argmax(runner.step([StepEntry(r, prompt, [len(prompt) - 1])])).tolist()[0])
    for _ in range(warmup):
        for r in range(batch):
            assert runner.reserve(r, 1)
        toks = ops.argmax(runner.step([StepEntry(r, [toks[r]], [0]) for r in range(batch)])).tolist()
    entries = [StepEntry(r, [0], [0]) for r in range(batch)]
    last = torch.tensor(toks, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ctx_sum, run = 0, []
    for r in range(batch):
        assert runner.reserve(r, steps)
    for _ in range(steps):
        ctx_sum += sum(runner.cached[r] + 1 for r in range(batch))
        last = ops.argmax(runner.step(entries, token_source=last))
        run.append(last)
    torch.stack(run).tolist()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for r in range(batch):
        runner.release(r)
    return dt, ctx_sum / steps


def prefill_run(runner, vocab: int, gen, t: int, runs: int = 4):
    """One request of ``t`` tokens, whole, ``runs`` times (the first warms up); the mean of the rest, in seconds."""
    import torch

    from yalis_amd.engine.step import StepEntry

    ops = runner.rt.ops
    prompt = torch.randint(0, vocab, (t,), generator=gen).tolist()
    times = []
    for i in range(runs):
        assert runner.admit(1000 + i) and runner.reserve(1000 + i, t)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ops.argmax(runner.step([StepEntry(1000 + i, prompt, [t - 1])])).tolist()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        runner.release(1000 + i)
    return sum(times[1:]) / len(times[1:]), times


def mixed_run(runner, shape: Shape, gen, prompt_len: int, portion: int, n_dec: int = 32, plen: int = 4096):
    """``n_dec`` requests decode while ``plen``-token prompts arrive in portions: every step holds
    ``n_dec`` single tokens and one portion (the last portion's row is sampled too).  The rows of
    a step's products are the step's tokens: 480 + 32 = 512 rows fill the vendor library's tiles,
    512 + 32 = 544 rows cost a fifth tile row for a quarter of its work.  Returns (ms a step,
    the bound max(bytes / HBM, flops / matrix cores) in ms, steps timed)."""
    import torch

    from yalis_amd.engine.step import StepEntry

    ops = runner.rt.ops
    toks = []
    for r in range(n_dec):
        assert runner.admit(r)
        prompt = torch.randint(0, shape.vocab, (prompt_len,), generator=gen).tolist()
        assert runner.reserve(r, len(prompt))
        toks.append(ops.argmax(runner.step([StepEntry(r, prompt, [len(prompt) - 1])])).tolist()[0])
    prompt = torch.randint(0, shape.vocab, (plen,), generator=gen).tolist()
    times, kv_tokens = [], []
    for rid in (100, 101, 102):  # the first prompt warms up
        assert runner.admit(rid)
        for c0 in range(0, plen - portion + 1, portion):
            for r in range(n_dec):
                assert runner.reserve(r, 1)
            assert runner.reserve(rid, portion)
            last = c0 + 2 * portion > plen
            entries = [StepEntry(r, [toks[r]], [0]) for r in range(n_dec)]
            entries.append(StepEntry(rid, prompt[c0 : c0 + portion], [portion - 1] if last else []))
            ctx_tokens = sum(runner.cached[r] + 1 for r in range(n_dec)) + c0 + portion
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = ops.argmax(runner.step(entries)).tolist()
            torch.cuda.synchronize()
            if rid != 100:
                times.append(time.perf_counter() - t0)
                kv_tokens.append(ctx_tokens)
            toks = out[:n_dec]
        runner.release(rid)
    for r in range(n_dec):
        runner.release(r)
    ms = 1e3 * sum(times) / len(times)
    n_tok = n_dec + portion
    step_b = shape.weight_bytes + sum(kv_tokens) / len(kv_tokens) * shape.kv_bytes_per_token
    # products over all tokens of the step; attention of the portion against the prompt so far
    step_f = shape.layers * (2 * n_tok * shape.layer_params + 4 * shape.h * shape.d * portion * (plen / 2)) + 2 * (n_dec + 1 / 8) * shape.vocab * shape.c
    bound_ms = 1e3 * max(step_b / (HBM_GBPS * 1e9), step_f / BF16_FLOPS)
    return ms, bound_ms, len(times)


def breakdown(runner, shape: Shape, gen, batch: int, prompt_len: int, prefill_len: int):
    """Where a decode step's and a prefill's time goes, by kind of work, from device events
    around every call into the kernel library (steps launched kernel by kernel for this: the
    replayed graph of a decode step cannot be timed from inside).  Each kind comes with what
    bounds it: products and the output head the bytes of their weights over the memory
    bandwidth (decode) or their flops over the matrix cores' rate (prefill), attention the bytes
    of the cached keys and values (decode) or its flops (prefill)."""
    import torch

    from yalis_amd.engine.step import StepEntry

    ops = runner.rt.ops
    kinds = {"linear": "products", "gate_up_act": "products", "gemm_mfma_skinny": None, "gemm_fma": None,
             "attention": "attention", "rope_append": "attention", "add_rmsnorm": "norms", "gather_add_rmsnorm": "norms",
             "gated_act": "activation", "embed": "other", "argmax": "other"}
    spans, depth, head_rows = [], [0], shape.vocab

    def timed(name, fn, kind):
        def call(*a, **kw):
            if depth[0]:  # a call made by a timed call belongs to it
                return fn(*a, **kw)
            k = kind
            if name == "linear" and a[1].shape[0] == head_rows:
                k = "head"
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            depth[0] += 1
            start.record()
            try:
                return fn(*a, **kw)
            finally:
                stop.record()
                depth[0] -= 1
                spans.append((k, start, stop))
        return call

    saved = {}
    for name, kind in kinds.items():
        if kind is not None and hasattr(ops, name):
            saved[name] = getattr(ops, name)
            setattr(ops, name, timed(name, saved[name], kind))
    graphs, runner.use_graphs = runner.use_graphs, False
    out = {}
    try:
        toks = []
        for r in range(batch):
            assert runner.admit(r)
            prompt = torch.randint(0, shape.vocab, (prompt_len,), generator=gen).tolist()
            assert runner.reserve(r, len(prompt) + 8)
            toks.append(ops.argmax(runner.step([StepEntry(r, prompt, [len(prompt) - 1])])).tolist()[0])
        sums, n_steps = {}, 4
        for i in range(n_steps + 2):
            spans.clear()
            toks = ops.argmax(runner.step([StepEntry(r, [toks[r]], [0]) for r in range(batch)])).tolist()
            torch.cuda.synchronize()
            if i >= 2:
                for k, a, b in spans:
                    sums[k] = sums.get(k, 0.0) + a.elapsed_time(b) * 1e3 / n_steps
        ctx = sum(runner.cached[r] for r in range(batch))
        for r in range(batch):
            runner.release(r)
        bytes_of = {"products": 2 * shape.layers * shape.layer_params, "attention": ctx * shape.kv_bytes_per_token, "head": 2 * shape.vocab * shape.c}
        out["decode_us"] = {k: round(v, 1) for k, v in sorted(sums.items())}
        out["decode_frac_of_hbm"] = {k: round(bytes_of[k] / (sums[k] * 1e-6) / (HBM_GBPS * 1e9), 3) for k in bytes_of if sums.get(k)}
        # prefill
        t = prefill_len
        prompt = torch.randint(0, shape.vocab, (t,), generator=gen).tolist()
        sums = {}
        for i in range(3):
            spans.clear()
            assert runner.admit(2000 + i) and runner.reserve(2000 + i, t)
            ops.argmax(runner.step([StepEntry(2000 + i, prompt, [t - 1])])).tolist()
            torch.cuda.synchronize()
            runner.release(2000 + i)
            if i >= 1:
                for k, a, b in spans:
                    sums[k] = sums.get(k, 0.0) + a.elapsed_time(b) / 2
        flops_of = {"products": 2 * t * shape.layers * shape.layer_params, "attention": 2 * shape.h * shape.d * t * t * shape.layers}
        out["prefill_ms"] = {k: round(v, 3) for k, v in sorted(sums.items())}
        out["prefill_frac_of_mfma"] = {k: round(flops_of[k] / (sums[k] * 1e-3) / BF16_FLOPS, 3) for k in flops_of if sums.get(k)}
    finally:
        runner.use_graphs = graphs
        for name, fn in saved.items():
            setattr(ops, name, fn)
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (both numbers are reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=1024)
    ap.add_argument("--prefill-len", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="the headline decode measurement only (no prefill, batch 1 / 64, breakdown, mixed steps)")
    ap.add_argument("--only-prefill", action="store_true", help="measure the prefill only (for profiling)")
    ap.add_argument("--mixed", action="store_true", help="measure mixed steps instead: 32 decode streams beside portions of 4,096-token prompts")
    ap.add_argument("--portion", type=int, default=480, help="tokens of a prompt portion in --mixed steps (with the 32 decoded tokens: 512 rows, as the scheduler cuts under a budget of 512)")
    ap.add_argument("--no-graphs", action="store_true", help="launch decode steps kernel by kernel (for hardware counters)")
    ap.add_argument("--shape", choices=("8b", "3b", "1b", "70b"), default="8b", help="layer sizes (default: the 8B shape of the headline)")
    ap.add_argument("--sample", action="store_true", help="time instead the choice of a token alone (greedy and each sampling rule) at the shape's vocabulary for --batch rows")
    ap.add_argument("--no-70b", action="store_true", help="leave out the points at the Llama-3.1-70B shape (decode at batch 1 / 8 / 64 behind 2,048-token prompts; 141 GB of weights)")
    ap.add_argument("--probe", action="store_true", help="measure instead what a plain streaming read and a plain matrix-core loop reach on this card")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single MI355X)")
        return 2

    import torch

    if args.probe:
        return machine_probe(SHAPES[args.shape][1])
    if args.sample:
        return sampling_times(SHAPES[args.shape][1]["vocab_size"], args.batch)

    shape_name, shape_cfg = SHAPES[args.shape]
    cfg = dict(shape_cfg)
    full_layers = cfg["num_hidden_layers"]
    if args.layers is not None:
        cfg["num_hidden_layers"] = args.layers
    shape = Shape(cfg)
    gen = torch.Generator().manual_seed(0)

    if args.mixed:
        runner = make_runner(cfg, 34, 4096 + 64, graphs=not args.no_graphs)
        ms, bound_ms, n = mixed_run(runner, shape, gen, args.prompt_len, args.portion)
        print(json.dumps({
            "metric": f"mixed steps ({shape_name} shape): 32 decode streams beside {args.portion}-token portions of 4,096-token prompts",
            "ms_per_step": round(ms, 3), "decode_tokens_per_s": round(32 / ms * 1e3, 1), "prefill_tokens_per_s": round(args.portion / ms * 1e3, 1),
            "steps": n, "dtype": "bf16", "n_gpus": 1,
            "roofline": {"bound": "max(hbm, mfma)", "bound_ms": round(bound_ms, 3), "frac": round(bound_ms / ms, 4)},
        }))
        return 0

    max_batch = max(args.batch, 1 if args.no_points else 64)
    total_steps = args.steps + args.warmup + 8
    ctx_cap = max(args.prompt_len + total_steps + 1, args.prefill_len)
    pool_tokens = 0
    further = not args.no_points and args.shape == "8b" and args.layers is None and not args.only_prefill
    if further:
        # further sizes: prompts of 8,192 tokens, batch 8 behind 8,000-token prompts, batch 64
        # behind 4,000-token ones (the pool holds the largest of them)
        ctx_cap = cfg["max_position_embeddings"]
        pool_tokens = 64 * (4000 + 64 + 64)
    engine = make_engine(cfg, max_batch, ctx_cap, graphs=not args.no_graphs, pool_tokens=pool_tokens)
    runner = engine.runner

    if args.only_prefill:
        _, times = prefill_run(runner, shape.vocab, gen, args.prefill_len, runs=3)
        for x in times:
            print(f"prefill {args.prefill_len} tokens: {1e3 * x:.3f} ms")
        return 0

    dt, mean_ctx = decode_run(runner, shape.vocab, gen, args.batch, args.prompt_len, args.steps, args.warmup)
    ms_per_step = 1e3 * dt / args.steps
    achieved = shape.decode_bytes(args.batch, mean_ctx) / (dt / args.steps) / 1e9
    result = {
        "metric": f"decode tok/s ({shape_name} shape, batch {args.batch}, {args.prompt_len:,}-token prompts)",
        "value": round(args.batch * args.steps / dt, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic: random N(0,0.02) bf16 weights, seeded uniform-random token ids",
        "config": {
            "model": f"{shape_name} shape",
            "layers": shape.layers,
            "layers_of_full_model": full_layers,
            "hidden_size": shape.c,
            "num_attention_heads": shape.h,
            "num_key_value_heads": shape.g,
            "head_dim": shape.d,
            "intermediate_size": shape.inter,
            "vocab_size": shape.vocab,
            "global_batch": args.batch,
            "seq_len": args.prompt_len,
            "context": cfg["max_position_embeddings"],
            "page_size": 64,
            "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_GBPS, 4)},
    }

    if not args.no_points:
        t = args.prefill_len
        pf, _ = prefill_run(runner, shape.vocab, gen, t, runs=4)  # the mean of three timed runs
        result["prefill"] = {"value": round(t / pf, 1), "tokens": t, "ms": round(1e3 * pf, 3),
                             "frac": round(shape.prefill_flops(t) / pf / BF16_FLOPS, 4)}
        points = {}
        for b, name in ((1, "decode_b1"), (64, "decode_b64")):
            steps = max(8, args.steps // 2)
            dtb, ctx_b = decode_run(runner, shape.vocab, gen, b, args.prompt_len, steps, 2)
            points[name] = round(b * steps / dtb, 2)
            # the same roofline as the headline: bytes the step has to read / its time / 8 TB/s
            points[name + "_frac"] = round(shape.decode_bytes(b, ctx_b) / (dtb / steps) / (HBM_GBPS * 1e9), 4)
        # the same workload through LLMEngine.generate itself: its own TTFT and TBT (scheduler,
        # sampler and the host's share included; the step-level figures above leave them out)
        gm = generate_metrics(engine, shape.vocab, gen, args.batch, args.prompt_len, args.steps + 1)
        points["generate_tbt_ms"] = round(gm["TBT"], 4)
        points["generate_ttft_ms"] = round(gm["TTFT"], 3)
        points["generate_tok_s"] = round(gm["Throughput"], 1)
        if further:
            for t2 in (512, 8192):
                pf2, _ = prefill_run(runner, shape.vocab, gen, t2, runs=3)
                points[f"prefill_{t2}_tok_s"] = round(t2 / pf2, 1)
                points[f"prefill_{t2}_frac"] = round(shape.prefill_flops(t2) / pf2 / BF16_FLOPS, 4)
            for b, plen, name in ((8, 8000, "decode_b8_ctx8k"), (64, 4000, "decode_b64_ctx4k")):
                dtb, ctx_b = decode_run(runner, shape.vocab, gen, b, plen, 8, 2)
                points[name] = round(b * 8 / dtb, 2)
                points[name + "_frac"] = round(shape.decode_bytes(b, ctx_b) / (dtb / 8) / (HBM_GBPS * 1e9), 4)
        result["breakdown"] = breakdown(runner, shape, gen, args.batch, args.prompt_len, t)
        del runner, engine
        torch.cuda.empty_cache()
        # mixed steps at the Llama-3.2-3B shape: 32 decode streams beside portions of 4,096-token
        # prompts, 512, 1,024 and 2,048 rows a step (only with the headline's own shape and all
        # its layers)
        if args.shape == "8b" and args.layers is None:
            name3, cfg3 = SHAPES["3b"]
            shape3 = Shape(cfg3)
            runner3 = make_runner(dict(cfg3), 34, 4096 + 64)
            for portion, tag in ((480, "mixed_3b"), (992, "mixed_3b_p992"), (2016, "mixed_3b_p2016")):
                ms3, bound3, _ = mixed_run(runner3, shape3, gen, args.prompt_len, portion)
                if portion == 480:
                    points["mixed_3b_ms_per_step"] = round(ms3, 3)
                    points["mixed_3b_decode_tok_s"] = round(32 / ms3 * 1e3, 1)
                    points["mixed_3b_prefill_tok_s"] = round(480 / ms3 * 1e3, 1)
                    points["mixed_3b_bound_ms"] = round(bound3, 3)  # max(bytes / 8 TB/s, flops / 2.5 PFLOP/s)
                else:
                    points[tag + "_ms_per_step"] = round(ms3, 3)
                    points[tag + "_prefill_tok_s"] = round(portion / ms3 * 1e3, 1)
                points[tag + "_frac"] = round(bound3 / ms3, 4)
            del runner3
            torch.cuda.empty_cache()
            if not args.no_70b and torch.cuda.mem_get_info()[0] > 200e9:
                # the Llama-3.1-70B shape (141 GB of weights on the one GPU), decode at batch 1, 8
                # and 64 behind 2,048-token prompts
                name70, cfg70 = SHAPES["70b"]
                shape70 = Shape(cfg70)
                runner70 = make_runner(dict(cfg70), 64, 2048 + 64)
                for b in (1, 8, 64):
                    dtb, ctx_b = decode_run(runner70, shape70.vocab, gen, b, 2048, 6, 2)
                    points[f"decode70b_b{b}"] = round(b * 6 / dtb, 2)
                    points[f"decode70b_b{b}_frac"] = round(shape70.decode_bytes(b, ctx_b) / (dtb / 6) / (HBM_GBPS * 1e9), 4)
                del runner70
                torch.cuda.empty_cache()
        result["points"] = points

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())

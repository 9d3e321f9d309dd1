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


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (both numbers are reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=1024)
    ap.add_argument("--prefill-len", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 and prefill measurements")
    ap.add_argument("--only-prefill", action="store_true", help="measure the prefill only (for profiling)")
    ap.add_argument("--mixed", action="store_true", help="measure mixed steps instead: 32 decode streams beside portions of 4,096-token prompts")
    ap.add_argument("--portion", type=int, default=480, help="tokens of a prompt portion in --mixed steps (with the 32 decoded tokens: 512 rows, as the scheduler cuts under a budget of 512)")
    ap.add_argument("--no-graphs", action="store_true", help="launch decode steps kernel by kernel (for hardware counters)")
    ap.add_argument("--shape", choices=("8b", "3b", "70b"), default="8b", help="layer sizes (default: the 8B shape of the headline)")
    ap.add_argument("--sample", action="store_true", help="time instead the choice of a token alone (greedy and each sampling rule) at the shape's vocabulary for --batch rows")
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

    from yalis_amd.config.runtime import EngineConfig
    from yalis_amd.engine.factory import random_runner
    from yalis_amd.engine.step import StepEntry

    shape_name, shape_cfg = SHAPES[args.shape]
    cfg = dict(shape_cfg)
    full_layers = cfg["num_hidden_layers"]
    if args.layers is not None:
        cfg["num_hidden_layers"] = args.layers
    layers = cfg["num_hidden_layers"]
    page = 64
    max_batch = max(args.batch, 1 if args.no_points else 64)
    total_steps = args.steps + args.warmup + 8
    ctx_cap = max(args.prompt_len + total_steps + 1, args.prefill_len)
    if args.mixed:
        max_batch, ctx_cap = 34, 4096 + 64
    pages_per_req = -(-ctx_cap // page)
    engine = EngineConfig(
        page_size=page,
        num_pages=pages_per_req * max_batch,
        max_num_seqs=max_batch,
        max_model_len=min(cfg["max_position_embeddings"], pages_per_req * page),
        max_num_batched_tokens=8192,
        dtype="bfloat16",
        decode_graphs=not args.no_graphs,
    )
    runner = random_runner(cfg, engine, seed=0)
    ops = runner.rt.ops
    vocab = cfg["vocab_size"]
    gen = torch.Generator().manual_seed(0)

    def decode_run(batch: int, steps: int, warmup: int):
        """Prefill ``batch`` prompts, then time ``steps`` decode steps."""
        for r in range(batch):
            assert runner.admit(r)
            prompt = torch.randint(0, vocab, (args.prompt_len,), generator=gen).tolist()
            assert runner.reserve(r, len(prompt))
            logits = runner.step([StepEntry(r, prompt, [len(prompt) - 1])])
            first = ops.argmax(logits).tolist()
            if r == 0:
                toks = []
            toks.append(first[0])

        def one_step(toks):
            for r in range(batch):
                assert runner.reserve(r, 1)
            logits = runner.step([StepEntry(r, [toks[r]], [0]) for r in range(batch)])
            return ops.argmax(logits).tolist()

        for _ in range(warmup):
            toks = one_step(toks)
        entries = [StepEntry(r, [0], [0]) for r in range(batch)]
        last = torch.tensor(toks, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ctx_sum = 0
        run = []
        for r in range(batch):
            assert runner.reserve(r, steps)
        for _ in range(steps):
            ctx_sum += sum(runner.cached[r] + 1 for r in range(batch))
            last = ops.argmax(runner.step(entries, token_source=last))
            run.append(last)
        toks = torch.stack(run).tolist()[-1]
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        for r in range(batch):
            runner.release(r)
        return dt, ctx_sum / steps  # seconds, mean cached tokens read per step

    c, h, g, d, inter = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["intermediate_size"]
    layer_params = c * (h + 2 * g) * d + h * d * c + 3 * c * inter
    # every weight a decode step reads once: the layers, the final norm, the output head (the
    # embedding table itself when tied; of a separate table only a row per token is read)
    weight_bytes = 2 * (layers * (layer_params + 2 * c) + c + vocab * c)

    def step_bytes(batch, mean_ctx_tokens):
        kv = mean_ctx_tokens * layers * 2 * g * d * 2
        return weight_bytes + batch * c * 2 + kv

    if args.mixed:
        # 32 requests decode while 4,096-token prompts arrive in portions: every step holds 32
        # single tokens and one portion (the last portion's row is sampled too).  The rows of a
        # step's products are the step's tokens: 480 + 32 = 512 rows fill the vendor library's
        # tiles, 512 + 32 = 544 rows cost a fifth tile row for a quarter of its work.
        n_dec, portion, plen = 32, args.portion, 4096
        toks = []
        for r in range(n_dec):
            assert runner.admit(r)
            prompt = torch.randint(0, vocab, (args.prompt_len,), generator=gen).tolist()
            assert runner.reserve(r, len(prompt))
            toks.append(ops.argmax(runner.step([StepEntry(r, prompt, [len(prompt) - 1])])).tolist()[0])
        prompt = torch.randint(0, vocab, (plen,), generator=gen).tolist()
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
        ms = 1e3 * sum(times) / len(times)
        n_tok = n_dec + portion
        mean_kv = sum(kv_tokens) / len(kv_tokens)
        step_b = weight_bytes + mean_kv * layers * 2 * g * d * 2
        # products over all tokens of the step; attention of the portion against the prompt so far
        step_f = layers * (2 * n_tok * layer_params + 4 * h * d * portion * (plen / 2)) + 2 * (n_dec + 1 / 8) * vocab * c
        bound_ms = 1e3 * max(step_b / (HBM_GBPS * 1e9), step_f / BF16_FLOPS)
        print(json.dumps({
            "metric": f"mixed steps ({shape_name} shape): {n_dec} decode streams beside {portion}-token portions of {plen:,}-token prompts",
            "ms_per_step": round(ms, 3), "decode_tokens_per_s": round(n_dec / ms * 1e3, 1), "prefill_tokens_per_s": round(portion / ms * 1e3, 1),
            "steps": len(times), "dtype": "bf16", "n_gpus": 1,
            "roofline": {"bound": "max(hbm, mfma)", "bound_ms": round(bound_ms, 3), "frac": round(bound_ms / ms, 4)},
        }))
        return 0

    if args.only_prefill:
        t = args.prefill_len
        prompt = torch.randint(0, vocab, (t,), generator=gen).tolist()
        for i in range(3):
            assert runner.admit(1000 + i) and runner.reserve(1000 + i, t)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ops.argmax(runner.step([StepEntry(1000 + i, prompt, [t - 1])])).tolist()
            torch.cuda.synchronize()
            print(f"prefill {t} tokens: {1e3 * (time.perf_counter() - t0):.3f} ms")
            runner.release(1000 + i)
        return 0

    dt, mean_ctx = decode_run(args.batch, args.steps, args.warmup)
    ms_per_step = 1e3 * dt / args.steps
    value = args.batch * args.steps / dt
    achieved = step_bytes(args.batch, mean_ctx) / (dt / args.steps) / 1e9

    result = {
        "metric": f"decode tok/s ({shape_name} shape, batch {args.batch}, {args.prompt_len:,}-token prompts)",
        "value": round(value, 2),
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
            "layers": layers,
            "layers_of_full_model": full_layers,
            "hidden_size": c,
            "num_attention_heads": h,
            "num_key_value_heads": g,
            "head_dim": d,
            "intermediate_size": inter,
            "vocab_size": vocab,
            "global_batch": args.batch,
            "seq_len": args.prompt_len,
            "context": cfg["max_position_embeddings"],
            "page_size": page,
            "parallelism": "single GPU",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_GBPS, 4),
        },
    }

    if not args.no_points:
        # prefill of one request of 2,048 tokens, whole
        t = args.prefill_len
        prompt = torch.randint(0, vocab, (t,), generator=gen).tolist()
        times = []
        for i in range(3):
            assert runner.admit(1000 + i)
            assert runner.reserve(1000 + i, t)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = runner.step([StepEntry(1000 + i, prompt, [t - 1])])
            ops.argmax(logits).tolist()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            runner.release(1000 + i)
        pf = min(times[1:])
        flops = layers * (2 * t * layer_params + 2 * h * d * t * t) + 2 * vocab * c
        result["prefill"] = {
            "value": round(t / pf, 1),
            "tokens": t,
            "ms": round(1e3 * pf, 3),
            "frac": round(flops / pf / BF16_FLOPS, 4),
        }
        points = {}
        for b, name in ((1, "decode_b1"), (64, "decode_b64")):
            steps = max(8, args.steps // 2)
            dtb, _ = decode_run(b, steps, 2)
            points[name] = round(b * steps / dtb, 2)
        result["points"] = points

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Command line in the manner of the reference's examples/infer.py (a script with its
settings at the top: model, prompts, tokens to generate, max batch size, precision,
top_p, temperature, ten timed ``generate`` calls, then the outputs; :13-124).  The same
settings are options here, under the reference's names.

    python -m yalis_amd.infer --model DIR --prompt-ids 1,2,3 --prompt-ids 4,5 \\
        --tokens-to-generate 32 --temperature 0 --precision bf16
"""
from __future__ import annotations

import argparse
import sys
from typing import List

import torch

# used when no prompt is given and the folder has a tokenizer (the reference's script has a
# list of its own built in, examples/infer.py:18-35)
DEFAULT_PROMPTS = [
    "Describe how a paged key-value cache hands out and takes back its pages.",
    "Why does decoding one token at a time read every weight of the model?",
    "Write a short note on what limits the speed of a matrix product with few rows.",
    "Name three things a scheduler must decide when the cache is full.",
]


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", "--model-path", dest="model_path", default=None, help="folder with config.json, model.safetensors (and a tokenizer for text prompts)")
    ap.add_argument("--random", dest="random_shape", default=None, metavar="SHAPE",
                    help="no folder: random weights (seed: --random-weights-seed, default 0) of a named shape: 8b, 3b, 1b, 70b, tiny-a, tiny-b")
    ap.add_argument("--model-name", default=None)
    ap.add_argument("--precision", "--dtype", dest="precision", default="bf16", choices=["bf16", "fp32", "bfloat16", "float32"])
    ap.add_argument("--prompt", action="append", default=[], help="a text prompt (repeatable; needs a tokenizer)")
    ap.add_argument("--prompt-ids", action="append", default=[], help="a prompt as comma-separated token ids (repeatable)")
    ap.add_argument("--random-prompts", default=None, metavar="N,LEN", help="N prompts of LEN seeded random token ids")
    ap.add_argument("--chat", action="store_true", help="wrap text prompts in the tokenizer's chat template (examples/infer.py:50-62 of the reference does)")
    ap.add_argument("--system-prompt", default=None, help="system message for --chat")
    ap.add_argument("--prompt-file", default=None, help="a file with one prompt a line: text, or comma-separated token ids")
    ap.add_argument("--tokens-to-generate", "--max-tokens", dest="tokens_to_generate", type=int, default=50)
    ap.add_argument("--max-batch-size", "--max-num-seqs", dest="max_batch_size", type=int, default=32)
    ap.add_argument("--max-length-of-generated-sequences", type=int, default=1024)
    ap.add_argument("--temperature", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=None)
    ap.add_argument("--top-p", type=float, default=0.80)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--iters", type=int, default=1, help="timed generate calls (the reference script runs 10)")
    ap.add_argument("--no-ignore-eos", action="store_true", help="stop a request at its EOS token")
    ap.add_argument("--ignore-eos", action="store_true", help="generate past EOS (the default, as in the reference)")
    ap.add_argument("--report-throughput", action="store_true")
    ap.add_argument("--random-weights-seed", type=int, default=None, help="ignore the folder's weights; random ones from this seed")
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--num-pages", type=int, default=None)
    ap.add_argument("--max-num-batched-tokens", "--max-batched-tokens", dest="max_num_batched_tokens", type=int, default=2048)
    ap.add_argument("--wide-tensors", choices=["auto", "keep", "cast"], default="auto",
                    help="what the bf16 engine does with tensors stored in 32 bits: auto (a checkpoint wholly in 32 bits is narrowed, "
                         "single wide tensors of a 16-bit checkpoint stay wide), keep, cast")
    ap.add_argument("--tune-library-products", action="store_true",
                    help="time the vendor library's candidates for new product shapes of up to 256 rows and keep the fastest "
                         "(results may then differ in their last bits from run to run)")
    args = ap.parse_args(argv)
    if (args.model_path is None) == (args.random_shape is None):
        ap.error("give either --model DIR or --random SHAPE")
    return args


def main(argv=None) -> int:
    args = parse_args(argv)
    from yalis_amd import InferenceConfig, LLMEngine, ModelConfig, print_rank0
    from yalis_amd.config.reader import read_config_json
    from yalis_amd.config.runtime import EngineConfig

    from yalis_amd.config.runtime import canonical_dtype

    inference_config = InferenceConfig(
        max_batch_size=args.max_batch_size,
        max_length_of_generated_sequences=args.max_length_of_generated_sequences,
        top_k=args.top_k,
        top_p=args.top_p,
        temperature=args.temperature,
        seed=args.seed,
    )
    if args.random_shape is not None:
        from yalis_amd.models.presets import shape

        label, raw = shape(args.random_shape)
        model_config = None
        print_rank0(f"Model = random weights of the {label} shape")
    else:
        model_config = ModelConfig(model_name=args.model_name, model_path=args.model_path, precision=args.precision)
        raw = read_config_json(args.model_path)
    engine_config = EngineConfig(
        page_size=args.page_size,
        num_pages=args.num_pages,
        max_num_seqs=args.max_batch_size,
        max_model_len=min(args.max_length_of_generated_sequences, int(raw.get("max_position_embeddings", 1 << 30))),
        max_num_batched_tokens=args.max_num_batched_tokens,
        dtype=canonical_dtype(args.precision),
        wide_tensors=args.wide_tensors,
        tune_library_products=args.tune_library_products,
    )
    if model_config is None:
        engine = LLMEngine.from_random(raw, inference_config, precision=args.precision, seed=args.random_weights_seed or 0,
                                       engine_config=engine_config)
    else:
        engine = LLMEngine(model_config, inference_config, engine_config=engine_config, random_weights_seed=args.random_weights_seed)

    prompts: List = []
    if args.prompt_ids:
        prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    elif args.random_prompts:
        n, length = (int(x) for x in args.random_prompts.split(","))
        g = torch.Generator().manual_seed(args.seed)
        vocab = engine.model.spec.vocab_size
        prompts = [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(n)]
    elif args.prompt_file:
        with open(args.prompt_file, encoding="utf-8") as f:
            lines = [ln.strip() for ln in f if ln.strip()]
        as_ids = all(all(t.strip().isdigit() for t in ln.split(",")) for ln in lines)
        prompts = [[int(t) for t in ln.split(",")] for ln in lines] if as_ids else lines
    elif args.prompt:
        prompts = list(args.prompt)
    elif engine.tokenizer is None:
        # nothing to tokenize text with: a few seeded random prompts instead of the built-in texts
        g = torch.Generator().manual_seed(args.seed)
        vocab = engine.model.spec.vocab_size
        prompts = [torch.randint(0, vocab, (16,), generator=g).tolist() for _ in range(min(4, args.max_batch_size))]
    else:
        prompts = DEFAULT_PROMPTS[: args.max_batch_size]
    if args.chat and prompts and isinstance(prompts[0], str):
        if engine.tokenizer is None or not getattr(engine.tokenizer, "chat_template", None):
            raise SystemExit("--chat needs a tokenizer with a chat template in the model folder")
        wrapped = []
        for p in prompts:
            conversation = ([{"role": "system", "content": args.system_prompt}] if args.system_prompt else []) + [{"role": "user", "content": p}]
            wrapped.append(engine.tokenizer.apply_chat_template(conversation, add_generation_prompt=True, tokenize=False))
        prompts = wrapped
    print_rank0(f"Number of prompts = {len(prompts)}")

    for _ in range(args.iters):
        output_tokens, metrics = engine.generate(
            prompts,
            tokens_to_generate=args.tokens_to_generate,
            report_throughput=True if args.iters > 1 else args.report_throughput,
            ignore_eos=not args.no_ignore_eos,
        )
    texts = None
    if engine.tokenizer is not None:
        texts = engine.tokenizer.batch_decode(output_tokens, skip_special_tokens=True)
    for i, prompt in enumerate(prompts):
        print_rank0("==========================\n")
        print_rank0(f"prompt = {prompt}")
        print_rank0(f"output = {texts[i] if texts is not None else output_tokens[i].tolist()}")
    print_rank0("==========================\n")
    print_rank0(f"metrics = {metrics}")
    return 0


if __name__ == "__main__":
    sys.exit(main())

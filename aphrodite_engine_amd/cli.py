"""Command line of the package's own engine.

  python -m aphrodite_engine_amd generate --model DIR --prompt-ids 5,17,3 [--prompt-ids ...] [--max-new-tokens N]
        [--dtype bfloat16|float32|float16] [--temperature T --top-k K --top-p P --seed S]
      token ids in, generated token ids out (one JSON line per prompt), through the scheduler and the sampler.

  python -m aphrodite_engine_amd trace --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N      (= bin/trace_run)
      replays a schedule read from standard input, one JSON object a line
          {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}
      all entries of a step run as ONE batch from the caches earlier steps left; the fp32 logits at the wanted places go
      to DIR/<step>.f32 ([wanted, vocab], little endian); 'done <step>' is printed after every step; requests named in
      'end' give their pages and state slot back.  Nothing is sampled.

The model class is chosen by config.json (registry.py).  Kernels that the model needs and the tree does not hold yet are
compiled on first use."""
import argparse
import json
import os
import sys

_DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32", "float16": "float16",
           "fp16": "float16"}


def _torch_dtype(name: str):
    import torch
    return getattr(torch, _DTYPES[name])


def _true_fp32() -> None:
    """float32 means float32: no reduced-precision matrix mode."""
    import torch
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")


def _engine(args, max_tokens: int, max_num_seqs: int):
    import torch
    from .engine import LLMEngine
    if not torch.cuda.is_available():
        raise SystemExit("no GPU: this engine has no CPU path")
    _true_fp32()
    return LLMEngine.from_pretrained(args.model, dtype=_torch_dtype(args.dtype), device="cuda", max_tokens=max_tokens,
                                     max_num_seqs=max_num_seqs, block_size=args.block_size,
                                     max_num_batched_tokens=args.max_num_batched_tokens)


def cmd_trace(args) -> int:
    import numpy as np
    import torch
    engine = _engine(args, args.max_tokens, args.max_num_seqs)
    os.makedirs(args.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = [(str(e["id"]), e["tokens"], e.get("want") or []) for e in step["entries"]]
        logits = engine.run_segments(entries) if entries else None
        if logits is not None and logits.shape[0] > 0:
            data = logits.to(torch.float32).cpu().numpy().astype("<f4")
            tmp = os.path.join(args.out, ".%s.part" % step["step"])
            data.tofile(tmp)
            os.replace(tmp, os.path.join(args.out, "%s.f32" % step["step"]))
        else:
            torch.cuda.synchronize()
        for rid in step.get("end") or []:
            if str(rid) in engine.requests:        # a request that never brought a token holds nothing
                engine.release(str(rid))
        sys.stdout.write("done %s\n" % step["step"])
        sys.stdout.flush()
    return 0


def cmd_generate(args) -> int:
    from .engine import SamplingParams
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    longest = max(len(p) for p in prompts) + args.max_new_tokens
    per = (longest + args.block_size - 1) // args.block_size * args.block_size
    seqs = min(len(prompts), args.max_num_seqs)
    engine = _engine(args, args.max_tokens or per * seqs, seqs)
    params = SamplingParams(max_tokens=args.max_new_tokens, temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                            seed=args.seed)
    for p, out in zip(prompts, engine.generate(prompts, params)):
        print(json.dumps({"prompt_token_ids": p, "token_ids": out}))
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="aphrodite_engine_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)

    def common(p):
        p.add_argument("--model", required=True, help="folder with config.json and *.safetensors")
        p.add_argument("--dtype", default="bfloat16", choices=sorted(_DTYPES))
        p.add_argument("--block-size", type=int, default=16)
        p.add_argument("--max-num-seqs", type=int, default=4, help="live requests (state slots)")
        p.add_argument("--max-num-batched-tokens", type=int, default=2048)
    t = sub.add_parser("trace", help="replay a schedule from standard input, write logits")
    common(t)
    t.add_argument("--out", required=True)
    t.add_argument("--max-tokens", type=int, required=True, help="tokens the page pool is made for")
    t.set_defaults(fn=cmd_trace)
    g = sub.add_parser("generate", help="generate from prompts given as token ids")
    common(g)
    g.add_argument("--prompt-ids", action="append", required=True, help="comma-separated token ids; repeatable")
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--max-tokens", type=int, default=0, help="page pool size in tokens (default: what the prompts need)")
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-k", type=int, default=-1)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=None)
    g.set_defaults(fn=cmd_generate)
    args = ap.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())

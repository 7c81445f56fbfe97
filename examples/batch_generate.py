"""Batched autoregressive generation with a sequence-mixer model (counterpart of spec_generate.py for the batch engine).

    python examples/batch_generate.py --model DIR [--dtype bfloat16|float16|float32] [--prompts "5 17 3" "9 9 1 4"]
                                      [--max-new-tokens 32] [--temperature 0.8 --topk 32 --topp 0.9 --seed 0]

DIR holds config.json (its "architecture" names the model class) and *.safetensors.  Prompts are token ids unless the
directory has tokenizer files.  Without --prompts, random ids of a few lengths are used.
"""
import argparse
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import __graft_entry__ as ge  # noqa: E402
from umbrella_amd.speculation.auto_engine import AutoEngine  # noqa: E402

ap = argparse.ArgumentParser()
ap.add_argument("--model", required=True)
ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float16", "float32"])
ap.add_argument("--prompts", nargs="*", default=None)
ap.add_argument("--max-new-tokens", type=int, default=32)
ap.add_argument("--max-batch", type=int, default=8)
ap.add_argument("--max-length", type=int, default=4096)
ap.add_argument("--temperature", type=float, default=0.0)
ap.add_argument("--topk", type=int, default=32)
ap.add_argument("--topp", type=float, default=0.9)
ap.add_argument("--seed", type=int, default=0)
args = ap.parse_args()

ge.build_seq()
engine = AutoEngine.from_config("cuda:0", engine="batch", model=args.model, dtype=getattr(torch, args.dtype),
                                max_length=args.max_length, max_batch=args.max_batch, temperature=args.temperature,
                                topk=args.topk, topp=args.topp, seed=args.seed)
engine.initialize()
if args.prompts:
    prompts = [engine.tokenizer.encode(p, return_tensors="pt").reshape(-1).tolist() for p in args.prompts]
else:
    g = torch.Generator().manual_seed(args.seed)
    prompts = [torch.randint(0, engine.vocab_size, (n,), generator=g).tolist() for n in (5, 23, 12, 64)]
for p, out in zip(prompts, engine.generate_batch(prompts, max_new_tokens=args.max_new_tokens)):
    print(f"prompt ({len(p)} tokens) -> {engine.tokenizer.decode(out)}")

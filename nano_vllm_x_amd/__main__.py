"""python -m nano_vllm_x_amd --model DIR --prompt-ids 5,17,3 [--max-new-tokens N] [--temperature T] [--dtype bfloat16|float16|float32]

Generate from one or more prompts with the model in DIR (config.json names the architecture; without a checkpoint the
weights are drawn from --seed).  Prompts are lists of token ids (--prompt-ids, repeatable) or text for the directory's
tokenizer (--prompt, repeatable); one JSON object per prompt is printed: its ids, the generated ids and, with a
tokenizer, their text."""
from __future__ import annotations

import argparse
import asyncio
import json


def main():
    ap = argparse.ArgumentParser(prog="python -m nano_vllm_x_amd")
    ap.add_argument("--model", required=True)
    ap.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids; may be given several times")
    ap.add_argument("--prompt", action="append", default=[], help="text for the model's tokenizer; may be given several times")
    ap.add_argument("--max-new-tokens", type=int, default=32)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--dtype", choices=("bfloat16", "float16", "float32"), default=None)
    ap.add_argument("--max-bs", type=int, default=8)
    ap.add_argument("--context-len", type=int, default=2048)
    ap.add_argument("--kv-cache-size", type=int, default=0, help="token slots of the pool (0: sized from free memory)")
    ap.add_argument("--enforce-eager", action="store_true")
    ap.add_argument("--seed", type=int, default=0)
    a = ap.parse_args()
    prompts = [[int(x) for x in p.split(",") if x.strip()] for p in a.prompt_ids] + list(a.prompt)
    if not prompts:
        ap.error("give at least one --prompt-ids or --prompt")

    from . import LLM, SamplingParams

    llm = LLM(a.model, max_bs=a.max_bs, context_len=a.context_len, kv_cache_size=a.kv_cache_size or None, enforce_eager=a.enforce_eager,
              dtype=a.dtype, seed=a.seed)

    async def one(prompt):
        ids = []
        sp = SamplingParams(temperature=a.temperature, top_k=a.top_k, top_p=a.top_p, max_new_tokens=a.max_new_tokens, ignore_eos=True,
                            eos_token_id=0)
        async for out in llm.generate(prompt, sp):
            ids.append(out.token_id)
        return ids

    async def run():
        return await asyncio.gather(*(one(p) for p in prompts))

    results = asyncio.run(run())
    for p, ids in zip(prompts, results):
        line = {"prompt": p, "generated_ids": ids}
        if llm.detokenize_stream:
            line["text"] = llm.detokenize([ids])[0]
        print(json.dumps(line), flush=True)
    llm.shutdown()


if __name__ == "__main__":
    main()

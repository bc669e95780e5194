"""Command line of the generate loop: ``python -m gbx_lm_amd.cli --model DIR ...``.

Works on token ids (``--prompt-ids 5,17,3``, repeatable) or, when the model folder has a tokenizer, on text (``--prompt``).
One prompt runs through ``generate_step`` (the one-sequence loop every model of the registry supports); several prompts run
together through ``BatchScheduler.generate`` for models that step ragged batches.  Sampling: greedy by default, ``--temp`` /
``--top-p`` / ``--seed`` build the sampler that both loops take (log-probabilities [n, vocab] -> token ids [n]).
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import Callable, List, Optional

import torch


def make_sampler(temp: float = 0.0, top_p: float = 1.0, seed: Optional[int] = None) -> Optional[Callable[[torch.Tensor], torch.Tensor]]:
    """None for greedy; else temperature sampling inside the smallest set of tokens whose probability reaches ``top_p``."""
    if temp <= 0.0:
        return None
    gen = torch.Generator()
    if seed is not None:
        gen.manual_seed(seed)

    def sample(logprobs: torch.Tensor) -> torch.Tensor:
        lp = (logprobs.float() / temp).cpu()
        lp = lp.reshape(-1, lp.shape[-1])
        probs = torch.softmax(lp, dim=-1)
        if top_p < 1.0:
            sp, si = torch.sort(probs, dim=-1, descending=True)
            keep = torch.cumsum(sp, dim=-1) - sp < top_p          # the token that crosses top_p stays
            sp = sp * keep
            probs = torch.zeros_like(probs).scatter_(-1, si, sp)
        tok = torch.multinomial(probs / probs.sum(-1, keepdim=True), 1, generator=gen).reshape(-1)
        return tok.to(logprobs.device)

    return sample


def main(argv: Optional[List[str]] = None) -> int:
    ap = argparse.ArgumentParser(description="Generate with a model folder (config.json + model*.safetensors)")
    ap.add_argument("--model", required=True)
    ap.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids; repeat for a batch")
    ap.add_argument("--prompt", action="append", default=[], help="text (needs a tokenizer in the model folder); repeat for a batch")
    ap.add_argument("--max-tokens", type=int, default=64)
    ap.add_argument("--temp", type=float, default=0.0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--stop-id", type=int, action="append", default=[], help="token id that ends a sequence")
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default=None, help="dense checkpoints: dtype of the matrix products")
    a = ap.parse_args(argv)

    from .utils import generate_step, load_model
    from .batching import BatchScheduler
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32, None: None}[a.dtype]
    model, config = load_model(a.model, dtype=dtype)
    tokenizer = None
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt_ids]
    if a.prompt:
        from .tokenizer_utils import load_tokenizer
        tokenizer = load_tokenizer(a.model, {}, eos_token_ids=config.get("eos_token_id", None))
        prompts += [tokenizer.encode(p) for p in a.prompt]
    if not prompts or any(not p for p in prompts):
        ap.error("give at least one non-empty --prompt-ids or --prompt")
    sampler = make_sampler(a.temp, a.top_p, a.seed)
    stop = set(a.stop_id)
    if len(prompts) == 1:
        out = []
        for tok, _, _ in generate_step(torch.tensor(prompts[0]), model, max_tokens=a.max_tokens, sampler=sampler):
            out.append(tok)
            if tok in stop:
                break
        outs = [out]
    else:
        if not hasattr(model, "forward_tokens"):
            ap.error("this model steps one sequence at a time: give one prompt")
        outs = BatchScheduler(model).generate(prompts, max_tokens=a.max_tokens, sampler=sampler, stop_tokens=stop)
    for p, o in zip(prompts, outs):
        line = {"prompt_tokens": len(p), "tokens": o}
        if tokenizer is not None:
            line["text"] = tokenizer.decode(o)
        print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

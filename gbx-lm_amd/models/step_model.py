"""What every model that steps ragged batches shares: the ``generate_step`` calling convention on top of ``forward_tokens``,
the per-run caches over one slot table, the last norm and output head.

A subclass builds ``self.model`` (with ``embed``, ``layers``, ``norm``) and implements ``forward_tokens(tokens [T], batch, caches)
-> fp32 stream [T, width]``.  ``layer_runs`` lists which layer each run of the stack uses (a layer may run more than once with
the same weights: every run has a cache of its own); ``model.layers`` is that list of runs, so a cache list is checked against
it as for any other model.
"""
from __future__ import annotations

from typing import Any, List

import torch
import torch.nn.functional as F
from torch import nn

from ..batching import StepBatch
from .cache import SequenceSlots


class RaggedStepModel(nn.Module):
    quantized = False                       # dense checkpoint: the loader skips the GBA strategy / re-initialisation

    def __init__(self, args):
        super().__init__()
        self.args = args
        self.model_type = args.model_type
        self.lm_head = nn.Linear(args.width, args.vocab, bias=False)
        self.lm_head.weight.requires_grad_(False)
        self.trace_layers = None            # a list collects the fp32 stream after every layer run (diagnostics, tests)

    @property
    def layer_runs(self) -> List[int]:
        return list(range(len(self.model.layers)))

    @property
    def layers(self):
        return [self.model.layers[i] for i in self.layer_runs]

    def required_kernels(self) -> None:
        """Load (and, in a checkout without built files, first compile) the one kernel library these models run on."""
        from .. import _lib
        _lib.mixers()

    def make_cache(self) -> List[Any]:
        """One cache per layer run over one shared slot table; slot 0 is handed to the one-sequence generate loop."""
        slots = SequenceSlots(1)
        slots.length[0] = 0
        return [layer.mixer.make_cache(slots) for layer in self.layers]

    def forward_tokens(self, tokens: torch.Tensor, batch: StepBatch, caches) -> torch.Tensor:
        raise NotImplementedError

    def logits(self, x: torch.Tensor) -> torch.Tensor:
        """Last norm and output head on rows of the stream."""
        w = self.lm_head.weight
        return F.linear(self.model.norm(x, w.dtype), w)

    def _run(self, inputs: torch.Tensor, cache):
        b, l = inputs.shape
        if cache is None:
            cache = self.make_cache()
            for _ in range(b - 1):
                cache[0].slots.acquire()
        slots = cache[0].slots
        if slots.n_slots < b or any(n < 0 for n in slots.length[:b]):
            raise ValueError("the cache does not hold a sequence for every row of the batch")
        batch = StepBatch.build(list(range(b)), [slots.length[s] for s in range(b)], [l] * b, inputs.device)
        x = self.forward_tokens(inputs.reshape(-1), batch, cache)
        for s in range(b):
            slots.length[s] += l
        return x

    def forward(self, inputs: torch.Tensor, mask=None, cache=None, hidden_states: bool = False):
        """[B, L] token ids, row b continuing sequence b of ``cache`` -> logits [B, L, vocab] (``generate_step`` convention)."""
        b, l = inputs.shape
        x = self._run(inputs, cache)
        logits = self.logits(x).view(b, l, -1)
        return (logits, x.view(b, l, -1)) if hidden_states else logits

    def last_logits(self, inputs: torch.Tensor, cache) -> torch.Tensor:
        """Logits of the last position only, [B, vocab]: the head never sees the prompt's other rows."""
        b, l = inputs.shape
        return self.logits(self._run(inputs, cache).view(b, l, -1)[:, -1])

    def prefill(self, inputs: torch.Tensor, cache) -> None:
        self._run(inputs, cache)

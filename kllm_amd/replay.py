"""Replaying a trace of steps through the engine's own step function.

A trace step names, per request, its next tokens and the places whose logits
are wanted, plus the requests that end after the step.  Nothing is sampled and
no scheduler is involved: the batch of each step is exactly what the trace
says.  This is the role the reference's oracle harness plays for its tests
(engine/oracle/oracle.go:83-134), made a program.
"""

from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np

from .engine import Engine, EngineOptions, StepEntry


class Replayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16,
                 device: int = 0, options: Optional[EngineOptions] = None):
        if options is None:
            # The pool holds max_tokens tokens; a request's count is rounded up
            # to whole pages (and to 64, which whole pages of 16 divide).
            options = EngineOptions(device=device, dtype=dtype, page_size=page_size,
                                    max_tokens=max_tokens, max_model_len=1 << 30,
                                    max_requests=64)
        self.engine = Engine.from_dir(model_dir, options)

    def step(self, entries: Sequence[dict], end: Sequence = ()) -> Optional[np.ndarray]:
        """Run one trace step; returns float32 logits [wanted, vocab] or None."""
        logits = None
        if entries:
            batch = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in entries]
            out = self.engine.step(batch)
            if out is not None:
                logits = out.detach().to("cpu").numpy().astype(np.float32, copy=False)
        for rid in end:
            if rid in self.engine.cache:
                self.engine.release(rid)
        return logits

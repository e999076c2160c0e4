"""Plain generation loops over the step function (reference: Model::generate,
engine/src/model.cpp:667-691 -- prefill, then argmax and a one-token step per
new token; the final token is never run through the model)."""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence

from ..csrc import ops
from .executor import Executor, StepEntry
from .model import load_model


def generate_greedy_on(executor: Executor, prompt: Sequence[int], n_new: int,
                       on_token: Optional[Callable[[int, int], None]] = None, request="generate") -> List[int]:
    """Greedy tokens for one prompt on an existing executor."""
    out: List[int] = []
    if n_new <= 0:
        return out
    executor.admit(request)
    try:
        logits = executor.step([StepEntry(request, list(prompt), [len(prompt) - 1])])
        for step in range(n_new):
            token = int(ops.argmax(logits)[0])
            out.append(token)
            if on_token is not None:
                on_token(step, token)
            if step + 1 < n_new:
                logits = executor.step([StepEntry(request, [token], [0])])
    finally:
        executor.release(request)
    return out


def generate_greedy(model_dir: str, prompt: Sequence[int], n_new: int, dtype="bfloat16",
                    device="cuda:0", page_tokens: int = 64) -> List[int]:
    model, _ = load_model(model_dir, dtype, device)
    total = len(prompt) + n_new
    executor = Executor(model, num_pages=-(-total // page_tokens), max_requests=1,
                        max_tokens=-(-total // page_tokens) * page_tokens, page_tokens=page_tokens)
    return generate_greedy_on(executor, prompt, n_new)

"""The generation loop over the step function.

Requests are token-id prompts.  They are taken in order, as many at a time as
the batch limit and the cache hold; a batch's prompts run in one step, then
every live sequence goes on by one token per step.  A sequence ends when it
has produced a stop token — which is part of its output, as in the
reference's program loop (/root/reference/core/src/model/gemma4_plan.cpp:1631-1637,
:1770-1774) — or ``max_tokens`` tokens; it then leaves the batch and its slot
goes back to the cache at once, while the others continue.  When a batch has
ended the next one starts, on the slots and pages the last one gave back.

The token at output index i of a sequence is drawn for absolute position
``prompt length + i`` (/root/reference/core/include/sonicboom/model/plan.h:217-221), so
with a seed a sequence's tokens are the same alone and in any batch.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Iterable, List, Optional, Sequence

from ..cache.paged import PAGE, pages_for
from ..sampling import Sampler, SamplingParams
from .step import StepEntry


@dataclass
class _Live:
    index: int                  # which request
    slot: int
    history: List[int]          # prompt + produced tokens
    prompt_len: int
    out: List[int] = field(default_factory=list)


def plan_batches(prompt_lens: Sequence[int], max_new: int, n_pages: int, max_batch: int,
                 max_slots: Optional[int] = None) -> List[List[int]]:
    """Split requests, in order, into batches the cache can hold to their ends.

    A request needs ``ceil((prompt + max_new) / PAGE)`` pages in the worst
    case (the last produced token is never fed back, but a page's rounding
    makes this bound simple and safe).  Raises ValueError for a request that
    does not fit an empty cache.
    """
    limit = max_batch if max_slots is None else min(max_batch, max_slots)
    if limit <= 0:
        raise ValueError("the batch limit must be positive")
    batches, cur, used = [], [], 0
    for i, n in enumerate(prompt_lens):
        if n <= 0:
            raise ValueError(f"request {i}: an empty prompt cannot be continued")
        need = pages_for(n + max_new)
        if need > n_pages:
            raise ValueError(
                f"request {i}: {n} prompt tokens + {max_new} new ones need {need} cache pages of {PAGE} "
                f"tokens, the cache has {n_pages}")
        if cur and (len(cur) >= limit or used + need > n_pages):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


def generate(engine, prompts: Sequence[Sequence[int]], params: SamplingParams = SamplingParams(),
             stop_tokens: Optional[Iterable[int]] = None, max_batch: int = 64,
             callback: Optional[Callable[[int, int], Optional[bool]]] = None,
             sampler=None,
             allowed: Optional[Callable[[int, Sequence[int]], Optional[bytes]]] = None) -> List[List[int]]:
    """Continue every prompt; returns the produced tokens per prompt.

    ``engine`` has ``alloc_slot()``, ``free_slot(slot)``, ``step(entries) ->
    logits`` and ``cache.n_pages`` / ``cache.max_slots``; when it also has
    ``decode_loop()`` the single-token steps go through that loop (fixed buffers,
    HIP graph replay, the choice, greedy or drawn, on the device inside the replayed step unless
    penalties or masks need the host).  ``stop_tokens``
    defaults to the model's own (its configuration's eos ids).  ``callback(i,
    token)`` is called for every produced token of request i in order; a true
    return value ends that request before that token, which is not part of the
    output (/root/reference/capi/src/capi.cpp:2892-2898: an abort at a token
    returns the tokens before it).  ``sampler`` has ``pick(logits, positions, histories)``
    and defaults to the device sampler for ``params``.  ``allowed(i, history)``, asked before
    every choice of request i, returns the bitmap of the ids it may choose from (bit i & 7 of
    byte i >> 3 for id i; None: any), the mask of constrained decoding; the sampler's ``pick``
    then gets the bitmaps as ``masks=``.  A request that may choose nothing ends there, as it
    does in the reference (/root/reference/capi/src/capi.cpp:2820).
    """
    params = params.validated()
    own_sampler = sampler is None
    sampler = sampler or Sampler(params)
    if stop_tokens is None:
        stop_tokens = getattr(getattr(engine, "model", None), "spec", None)
        stop_tokens = stop_tokens.stop_tokens if stop_tokens is not None else ()
    stop = frozenset(int(t) for t in stop_tokens)
    prompts = [list(map(int, p)) for p in prompts]
    outputs: List[List[int]] = [[] for _ in prompts]
    if params.max_tokens == 0 or not prompts:
        return outputs
    # a bound on positions (the model's own unless the engine was given another; 0 = none): a prompt
    # beyond it is refused, a sequence that reaches it ends there
    max_positions = int(getattr(engine, "max_positions", 0) or 0)
    for i, p in enumerate(prompts):
        if max_positions and len(p) > max_positions:
            raise ValueError(f"request {i}: a prompt of {len(p)} tokens passes the model's {max_positions} positions")
    batches = plan_batches([len(p) for p in prompts], params.max_tokens, engine.cache.n_pages, max_batch,
                           engine.cache.max_slots)
    loop = engine.decode_loop() if hasattr(engine, "decode_loop") else None
    # the choice inside the loop's recorded step: greedy, or a draw that needs nothing of the host
    on_device = loop is not None and own_sampler and not params.has_penalties and allowed is None
    draw = sampler.device_draw(engine.model.vocab) if on_device else None

    def pick(logits, live):
        more = {} if allowed is None else {"masks": [allowed(s.index, s.history) for s in live]}
        return sampler.pick(logits, [len(s.history) for s in live], [s.history for s in live], **more)

    for batch in batches:
        live = [_Live(i, engine.alloc_slot(), list(prompts[i]), len(prompts[i])) for i in batch]
        try:
            # The prompts in one step; logits of every last row.
            logits = engine.step([StepEntry(s.slot, prompts[s.index], (s.prompt_len - 1,)) for s in live])
            tokens = pick(logits, live)
            started = False
            while True:
                flags = []
                for s, t in zip(live, tokens):
                    t = int(t)
                    if t < 0:
                        ended = True                     # nothing could be chosen
                    elif callback is not None and callback(s.index, t):
                        ended = True                     # aborted at this token: it is not reported
                    else:
                        s.out.append(t)
                        s.history.append(t)
                        ended = t in stop or len(s.out) >= params.max_tokens or \
                            (max_positions > 0 and len(s.history) > max_positions)
                    if ended:
                        outputs[s.index] = s.out
                        engine.free_slot(s.slot)
                        s.slot = -1
                    flags.append(not ended)
                fed = [int(t) for t, k in zip(tokens, flags) if k]
                live = [s for s, k in zip(live, flags) if k]
                if not live:
                    break
                # every live sequence goes on by the token it has just produced
                if loop is None:
                    logits = engine.step([StepEntry(s.slot, (t,), (0,)) for s, t in zip(live, fed)])
                    tokens = pick(logits, live)
                    continue
                if not started or not all(flags):
                    loop.start([s.slot for s in live], fed)
                    started = True
                if on_device:
                    tokens = loop.step(draw)         # the choice on the device, fed back by the loop
                else:
                    logits = loop.step_logits(fed)
                    tokens = pick(logits, live)
        finally:
            for s in live:
                if s.slot >= 0:
                    engine.free_slot(s.slot)
                    s.slot = -1
    return outputs

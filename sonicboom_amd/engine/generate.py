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
                 max_slots: Optional[int] = None, held: Optional[Sequence[int]] = None) -> List[List[int]]:
    """Split requests, in order, into batches the cache can hold to their ends.

    A request needs ``ceil((prompt + max_new) / PAGE)`` pages in the worst
    case (the last produced token is never fed back, but a page's rounding
    makes this bound simple and safe).  ``held[i]``: pages that request i
    already holds in a kept sequence (0: none); they, and that sequence's slot,
    stay taken while earlier batches run.  Raises ValueError for a request that
    does not fit.
    """
    if max_batch <= 0 or (max_slots is not None and max_slots <= 0):
        raise ValueError("the batch limit must be positive")
    held = [0] * len(prompt_lens) if held is None else list(held)
    later_pages = [0] * (len(held) + 1)          # pages and slots that requests after i hold already
    later_slots = [0] * (len(held) + 1)
    for i in range(len(held) - 1, -1, -1):
        later_pages[i] = later_pages[i + 1] + held[i]
        later_slots[i] = later_slots[i + 1] + (1 if held[i] else 0)
    batches, cur, used = [], [], 0
    for i, n in enumerate(prompt_lens):
        if n <= 0:
            raise ValueError(f"request {i}: an empty prompt cannot be continued")
        need = pages_for(n + max_new)
        room = n_pages - later_pages[i + 1]
        limit = max_batch if max_slots is None else min(max_batch, max_slots - later_slots[i + 1])
        if need > room or limit <= 0:
            raise ValueError(
                f"request {i}: {n} prompt tokens + {max_new} new ones need {need} cache pages of {PAGE} "
                f"tokens, the cache has {n_pages}" + (f" ({later_pages[i + 1]} held by kept sequences of "
                                                     f"later requests)" if later_pages[i + 1] else ""))
        if cur and (len(cur) >= limit or used + need > room):
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
             allowed: Optional[Callable[[int, Sequence[int]], Optional[bytes]]] = None,
             kept=None) -> List[List[int]]:
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
    does in the reference (/root/reference/capi/src/capi.cpp:2820).  ``kept`` (a
    :class:`~sonicboom_amd.engine.prefix.KeptSequences` of this engine): every request leaves its
    sequence in the cache when it ends, and a prompt that starts like a sequence the last call
    left feeds only what is new (``kept.reused[i]`` tokens of request i are not fed again); the
    produced tokens are the same either way.
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
    matches = [None] * len(prompts)
    if kept is not None:
        matches = kept.match(prompts)          # the matched slots are cut to the shared prefix
        kept.drop_all()                        # what no prompt continues goes back to the cache
    held_slots = {m[0] for m in matches if m}
    try:
        try:
            batches = plan_batches([len(p) for p in prompts], params.max_tokens, engine.cache.n_pages, max_batch,
                                   engine.cache.max_slots,
                                   [len(engine.cache.page_table(0, [m[0]])[0]) if m and engine.cache.groups else 0
                                    for m in matches])
        except ValueError:
            if not held_slots:
                raise
            # the kept sequences of later requests leave an earlier one no room: go without them
            for slot in held_slots:
                engine.free_slot(slot)
            held_slots.clear()
            matches = [None] * len(prompts)
            kept.reused = [0] * len(prompts)
            batches = plan_batches([len(p) for p in prompts], params.max_tokens, engine.cache.n_pages, max_batch,
                                   engine.cache.max_slots)
    except BaseException:
        for slot in held_slots:
            engine.free_slot(slot)
        raise
    loop = engine.decode_loop() if hasattr(engine, "decode_loop") else None
    # the choice inside the loop's recorded step: greedy, or a draw that needs nothing of the host
    on_device = loop is not None and own_sampler and not params.has_penalties and allowed is None
    draw = sampler.device_draw(engine.model.vocab) if on_device else None

    def pick(logits, live):
        more = {} if allowed is None else {"masks": [allowed(s.index, s.history) for s in live]}
        return sampler.pick(logits, [len(s.history) for s in live], [s.history for s in live], **more)

    def end(s):
        """The request's sequence leaves the batch: its slot is kept with its tokens, or freed."""
        slot, s.slot = s.slot, -1
        held_slots.discard(slot)
        if kept is not None:
            kept.put(slot, s.history[:engine.length(slot)])     # the last produced token is not in the cache
        else:
            engine.free_slot(slot)

    for batch in batches:
        live = []
        try:
            if kept is not None and len(kept):
                # sequences that earlier batches of this call have left make room for this one
                held_now = sum(len(engine.cache.page_table(0, [matches[i][0]])[0]) for i in batch
                               if matches[i] and engine.cache.groups)
                kept.make_room(sum(pages_for(len(prompts[i]) + params.max_tokens) for i in batch) - held_now,
                               sum(1 for i in batch if not matches[i]))
            for i in batch:
                slot = matches[i][0] if matches[i] else engine.alloc_slot()
                live.append(_Live(i, slot, list(prompts[i]), len(prompts[i])))
            # The prompts in one step (of a kept sequence only what is new); logits of every last row.
            skip = [matches[s.index][1] if matches[s.index] else 0 for s in live]
            logits = engine.step([StepEntry(s.slot, prompts[s.index][k:], (s.prompt_len - k - 1,))
                                  for s, k in zip(live, skip)])
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
                        end(s)
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
        except BaseException:
            for slot in held_slots - {s.slot for s in live}:       # kept sequences of batches that never ran
                engine.free_slot(slot)
            held_slots.intersection_update({s.slot for s in live})
            raise
        finally:
            for s in live:
                if s.slot >= 0:
                    held_slots.discard(s.slot)
                    engine.free_slot(s.slot)
                    s.slot = -1
    return outputs

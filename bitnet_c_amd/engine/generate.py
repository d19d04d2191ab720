"""The generation loop above the step function.

Requests are served in batches that start together: the prompts of a batch (unequal
lengths) run in one step, then every live sequence gets one token per step; a sequence
that samples a stop token, reaches its budget or the sequence limit leaves the batch and
gives its slot back at once, the others go on; when a batch is empty the next requests
form the next batch, until none is left.

Per sequence the order is the reference's (src/generate.c:156-229): sample from the
logits that are ready -> a stop token ends the sequence and is not emitted -> the token
is emitted (the callback may cancel) -> when the budget is reached no further step runs
-> otherwise the token is fed for the next logits.  Its loop detector, stop strings and
chat templates are serving helpers and are not taken over.

Decode steps are queued one ahead of the host where that is possible: when the sampler can
leave its tokens on the device (`sample_fn.start(logits, samplers)` returns an object with
device_tokens, rows(indices) and tokens(), or None when it needs the host first) and the engine
takes them from there (`takes_device_tokens`, step(entries, device_tokens=...)), the next step
is queued for every sequence that neither its budget nor the sequence limit ends, before the
host has seen the tokens.  It then reads them and decides as above; a sequence that its token
has ended (a stop token, a cancelling callback) has run one step for nothing, and its row of
the new logits is dropped.  The device so never waits for the host between two steps; tokens,
their order and the finish reasons are the same either way.

Nothing here touches the GPU directly: `engine` needs new_sequence(), release(slot),
step(entries) -> logits, max_seq_len and a cache that can tell how many tokens fit, and
`sample_fn(logits, samplers)` picks the tokens, so the decisions run in tests with stand-ins.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

from ..cache import PAGE
from ..sampling.sampler import SamplingParams, SequenceSampler
from .step import StepEntry, StepError


@dataclass
class Request:
    prompt: Sequence[int]
    max_new_tokens: int = 256
    params: SamplingParams = field(default_factory=SamplingParams)
    stop_ids: Sequence[int] = ()


@dataclass
class Result:
    tokens: List[int] = field(default_factory=list)
    finish: str = ""          # "stop" | "length" | "limit" | "cancelled" | "error: ..."
    prompt_len: int = 0


@dataclass
class _Live:
    index: int
    slot: int
    req: Request
    sampler: SequenceSampler
    length: int               # tokens in the cache


def _tokens_needed(req: Request, max_seq_len: int) -> int:
    n = min(len(req.prompt) + max(req.max_new_tokens, 0), max_seq_len)
    return ((n + PAGE - 1) // PAGE) * PAGE


def plan_batches(requests: Sequence[Request], batch_size: int, max_tokens: int, max_seq_len: int):
    """Cut the requests, in order, into batches of at most batch_size whose token needs
    (each rounded up to a page) fit max_tokens together.  Returns (batches, errors): lists of
    request indices, and index -> message for requests that can never run."""
    batches, errors, cur, used = [], {}, [], 0
    for i, r in enumerate(requests):
        if len(r.prompt) == 0:
            errors[i] = "error: empty prompt"
            continue
        if len(r.prompt) > max_seq_len:
            errors[i] = f"error: prompt of {len(r.prompt)} tokens exceeds the sequence limit {max_seq_len}"
            continue
        need = _tokens_needed(r, max_seq_len)
        if need > max_tokens:
            errors[i] = f"error: the request needs {need} cached tokens, the cache holds {max_tokens}"
            continue
        if cur and (len(cur) >= batch_size or used + need > max_tokens):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches, errors


def generate(engine, requests: Sequence[Request], sample_fn: Callable, batch_size: int = 8,
             on_token: Optional[Callable[[int, int], bool]] = None,
             max_tokens: Optional[int] = None) -> List[Result]:
    results = [Result(prompt_len=len(r.prompt)) for r in requests]
    cap = max_tokens if max_tokens is not None else engine.cache.n_pages * PAGE
    batches, errors = plan_batches(requests, batch_size, cap, engine.max_seq_len)
    for i, msg in errors.items():
        results[i].finish = msg
    prepare = getattr(engine, "prepare_decode", None)
    # a sampler that can leave its tokens on the device and an engine that takes them from there: decode steps are
    # queued one ahead of the tokens that the host has seen
    start = getattr(sample_fn, "start", None) if getattr(engine, "takes_device_tokens", False) else None
    for batch in batches:
        live: List[_Live] = []
        if prepare is not None and any(requests[i].max_new_tokens > 1 for i in batch):
            prepare(len(batch))          # whatever the decode steps will need is made now, not between two tokens
        try:
            for i in batch:
                r = requests[i]
                live.append(_Live(i, engine.new_sequence(), r, SequenceSampler(r.params, r.prompt), 0))
            # the prompts, in one step; logits at each prompt's last token
            logits = engine.step([StepEntry(s.slot, list(s.req.prompt), [len(s.req.prompt) - 1]) for s in live])
            for s in live:
                s.length = len(s.req.prompt)
            while live:
                done_now = [s for s in live if s.req.max_new_tokens <= 0]
                for s in done_now:
                    results[s.index].finish = "length"
                if done_now:
                    keep = [k for k, s in enumerate(live) if s.req.max_new_tokens > 0]
                    logits = logits[keep] if keep else logits[:0]
                    for s in done_now:
                        engine.release(s.slot)
                    live = [s for s in live if s.req.max_new_tokens > 0]
                    if not live:
                        break
                samplers = [s.sampler for s in live]
                pending = start(logits, samplers) if start is not None else None
                ahead = None
                if pending is not None:
                    # Whoever is neither at its budget nor at the limit goes on unless its token ends it.  The host
                    # learns that a step late: the next step is queued for all of them on the tokens that lie on the
                    # device, and a sequence that its token has ended leaves it unused.
                    cont = [k for k, s in enumerate(live)
                            if len(results[s.index].tokens) + 1 < s.req.max_new_tokens and s.length + 1 <= engine.max_seq_len]
                    if cont:
                        toks = pending.device_tokens if len(cont) == len(live) else pending.rows(cont)
                        try:
                            ahead = (cont, engine.step([StepEntry(live[k].slot, [0], [0]) for k in cont], device_tokens=toks))
                        except StepError:
                            ahead = None             # nothing has changed: decided below, with the tokens at hand
                    tokens = pending.tokens()
                else:
                    tokens = sample_fn(logits, samplers)
                nxt: List[int] = []
                for k, (s, tok) in enumerate(zip(live, tokens)):
                    res = results[s.index]
                    if tok in s.req.stop_ids:
                        res.finish = "stop"                      # not emitted
                    else:
                        res.tokens.append(int(tok))
                        s.sampler.accept(tok)
                        if on_token is not None and on_token(s.index, int(tok)):
                            res.finish = "cancelled"
                        elif len(res.tokens) >= s.req.max_new_tokens:
                            res.finish = "length"                # no further step for it
                        elif s.length + 1 > engine.max_seq_len:
                            res.finish = "limit"
                    if res.finish:
                        engine.release(s.slot)
                    else:
                        nxt.append(k)
                if ahead is not None:
                    cont, logits = ahead
                    if len(nxt) != len(cont):                    # rows of sequences that their token has ended
                        row_of = {k: r for r, k in enumerate(cont)}
                        logits = logits[[row_of[k] for k in nxt]]
                live = [live[k] for k in nxt]
                if not live:
                    break
                if ahead is None:
                    logits = engine.step([StepEntry(s.slot, [results[s.index].tokens[-1]], [0]) for s in live])
                for s in live:
                    s.length += 1
        except Exception:
            for s in live:
                if not results[s.index].finish:
                    try:
                        engine.release(s.slot)
                    except Exception:
                        pass
            raise
    return results

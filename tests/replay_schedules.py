"""Schedules that replay the same requests in different cuts through a `ReplaySession`, for a
model folder and a plain implementation of its architecture: whole, with a decoded tail, in
portions of changing size, token by token from the first, and mixed four at a time in a pool
that is used again.  Every schedule compares all logits with the plain implementation's."""

from __future__ import annotations

import torch

from tests import helpers

F32 = dict(atol=2e-5, rtol=2e-5)
LENGTHS = {"a": 150, "b": 97, "c": 64, "d": 41, "e": 33, "f": 5}
PORTIONS = [16, 7, 2, 5, 3, 2, 33, 2, 64, 9, 2, 17]


def entry(key, tokens):
    return {"id": key, "tokens": tokens, "want": list(range(len(tokens)))}


def check(got, want, dtype, what, bf16_cost):
    """float32: at float32 tolerances relative to the size of the logits.  bfloat16: within
    1.5 times `bf16_cost`, what the format costs the plain implementation on the same input
    at its worst position."""
    assert got.shape == want.shape, f"{what}: {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    diff = (got - want).abs()
    if dtype == "bfloat16":
        bound = torch.full_like(want, 1.5 * bf16_cost)
    else:
        bound = F32["atol"] * max(1.0, float(want.abs().max())) + F32["rtol"] * want.abs()
    bad = (diff > bound).any(-1)
    if bad.any():
        first = int(bad.nonzero()[0])
        raise AssertionError(
            f"{what}: worst difference {diff.max().item():.3e} (bound {bound.max().item():.3e}), "
            f"first wrong token {first} of {got.shape[0]}, {int(bad.sum())} wrong")


SCALES = (1.0, 1.31, 0.77, 1.73, 0.59, 1.13)


def position_error(x, want):
    """[T]: the root mean square over the vocabulary of the difference of the logits, the mean
    taken off."""
    d = x - want
    return (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt()


def rounding_cost(plain, cfg, weights, tokens, want):
    """[T]: what bfloat16 roundings between the products cost the plain implementation at each
    position, the largest of several runs whose roundings fall differently (the tensors are
    scaled by a factor that is no power of two before they are rounded, and back).  One run
    is one draw of the rounding errors; a position where a small error is made large (a head's
    output that nearly cancels before it is divided by its own size, the first tokens of a
    recurrence whose state holds one or two terms, a choice of experts that is a close call)
    shows in some of the draws."""
    costs = []
    for c in SCALES:
        r = plain.to_bf16 if c == 1.0 else (lambda t, c=c: plain.to_bf16(t * c) / c)
        costs.append(position_error(plain.forward(cfg, weights, tokens, r), want))
    return torch.stack(costs).max(0).values


def check_positions(got, want, cost, what):
    """bfloat16, position by position: the engine's error at a position may be 3 times
    `cost` there (or at the median position, where that is more).  One position in 25 may be
    over (a decision that rounding turned in the engine and in none of the plain runs), one in
    50 by more than half; the median position is within 1.5 times the plain's."""
    assert got.shape == want.shape and torch.isfinite(got).all(), what
    error = position_error(got, want)
    ratio = error / (3.0 * torch.maximum(cost, cost.median()))
    n = got.shape[0]
    over, far = int((ratio > 1).sum()), int((ratio > 1.5).sum())
    assert over <= max(1, n // 25) and far <= max(1, n // 50), (
        f"{what}: {over} of {n} positions over ({far} by more than half), the worst "
        f"{ratio.max():.2f} times its allowance (position {int(ratio.argmax())})")
    assert error.median() <= 1.5 * cost.median(), f"{what}: the median position"


class Case:
    """A model folder, six requests of LENGTHS, and what the plain implementation says of them
    (in float64, and what bfloat16 roundings cost it).  A plain implementation with a
    `pick_tokens(cfg, weights, count, seed)` chooses the requests' tokens itself (so that no
    position's decisions, a choice of experts for one, are a close call that bfloat16 rounding
    may decide the other way)."""

    def __init__(self, name, folder, page, plain, lengths=None):
        self.name, self.folder, self.page, self.plain = name, folder, page, plain
        self.cfg = plain.read_config(folder)
        self.weights = plain.read_weights(folder)
        pick = getattr(plain, "pick_tokens", None)
        self.reqs = {k: pick(self.cfg, self.weights, n, ord(k)) if pick
                     else helpers.random_tokens(self.cfg["vocab"], n, seed=ord(k))
                     for k, n in (lengths or LENGTHS).items()}
        exact = plain.read_weights(folder, torch.float64)
        self.want = {k: plain.forward(self.cfg, exact, v).float() for k, v in self.reqs.items()}
        self.cost = {k: rounding_cost(plain, self.cfg, self.weights, v, self.want[k])
                     for k, v in self.reqs.items()}

    def session(self, dtype, max_tokens, max_live=4):
        from mercury_amd.engine.replay import ReplaySession

        return ReplaySession(self.folder, dtype, max_tokens, page_size=self.page, max_live=max_live)

    def check(self, got, key, dtype, what, rows=None):
        want = self.want[key] if rows is None else self.want[key][rows]
        if dtype == "bfloat16":
            cost = self.cost[key] if rows is None else self.cost[key][rows]
            check_positions(got, want, cost, f"{self.name} {what} {key}")
        else:
            check(got, want, dtype, f"{self.name} {what} {key}", 0.0)


def whole(model, dtype):
    s = model.session(dtype, 192)
    for key, tokens in model.reqs.items():
        got = s.step([entry(key, tokens)], [key])
        model.check(got, key, dtype, "whole")
    assert s.manager.leaked_pages() == 0


def decoded_tail(model, dtype, keys=("a", "d", "e"), tail=32):
    s = model.session(dtype, 192)
    for key in keys:
        tokens = model.reqs[key]
        head = len(tokens) - tail
        rows = [s.step([entry(key, tokens[:head])], [])]
        for i in range(head, len(tokens)):
            rows.append(s.step([entry(key, tokens[i:i + 1])], [key] if i == len(tokens) - 1 else []))
        model.check(torch.cat(rows), key, dtype, "tail-decode")
    assert s.manager.leaked_pages() == 0


def portions(model, dtype, keys=("a", "b", "c")):
    s = model.session(dtype, 192)
    for shift, key in enumerate(keys):
        tokens, done, rows, n = model.reqs[key], 0, [], shift
        while done < len(tokens):
            count = min(PORTIONS[n % len(PORTIONS)], len(tokens) - done)
            n += 1
            last = done + count == len(tokens)
            rows.append(s.step([entry(key, tokens[done:done + count])], [key] if last else []))
            done += count
        model.check(torch.cat(rows), key, dtype, "portions")
    assert s.manager.leaked_pages() == 0


def from_the_first_token(model, dtype, key="a"):
    s = model.session(dtype, 192)
    tokens = model.reqs[key]
    rows = [s.step([entry(key, tokens[i:i + 1])], [key] if i == len(tokens) - 1 else [])
            for i in range(len(tokens))]
    model.check(torch.cat(rows), key, dtype, "decode-from-0")
    assert s.manager.leaked_pages() == 0


def mixed(model, dtype, order=("a", "d", "e", "b", "f", "c", "d", "a", "f", "e")):
    """Up to four live requests over four state slots, portions of some beside single tokens of
    others; the pool holds one long and a few short requests, so that pages and slots are given
    back and taken again.  Some requests run twice."""
    unit = max(64, model.page)
    live_cap = 5 * unit
    s = model.session(dtype, live_cap, max_live=4)
    order = list(order)
    got = {i: [] for i in range(len(order))}
    done = {i: 0 for i in range(len(order))}
    waiting, live, n = list(range(len(order))), [], 0
    rounded = lambda i: -(-len(model.reqs[order[i]]) // unit) * unit
    while waiting or live:
        while waiting and len(live) < 4 and sum(map(rounded, live)) + rounded(waiting[0]) <= live_cap:
            live.append(waiting.pop(0))
        entries, ends = [], []
        for slot, i in enumerate(list(live)):
            tokens = model.reqs[order[i]]
            left = len(tokens) - done[i]
            # the oldest request decodes token by token once it is past its first half; the
            # newest sits out every third step
            if slot == len(live) - 1 and len(live) > 1 and n % 3 == 2:
                n += 1
                continue
            count = 1 if (slot == 0 and done[i] > len(tokens) // 2) else PORTIONS[n % len(PORTIONS)]
            n += 1
            count = min(count, left)
            entries.append((i, {"id": f"r{i}", "tokens": tokens[done[i]:done[i] + count],
                                "want": list(range(count))}))
            done[i] += count
            if done[i] == len(tokens):
                ends.append(f"r{i}")
                live.remove(i)
        out = s.step([e for _, e in entries], ends)
        at = 0
        for i, e in entries:
            got[i].append(out[at:at + len(e["tokens"])])
            at += len(e["tokens"])
    for i, key in enumerate(order):
        model.check(torch.cat(got[i]), key, dtype, f"mixed (request {i})")
    assert s.manager.leaked_pages() == 0

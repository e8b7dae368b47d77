"""Schedules for replay tests, in the line format ``bin/trace_run`` reads, and
helpers that drive a Runner with them and sort the logits by request and position."""

from __future__ import annotations

import numpy as np
import torch


def whole(requests: dict[str, list[int]]) -> list[dict]:
    """Each request alone and whole: one step, every position wanted."""
    steps = []
    for rid, tokens in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": tokens, "want": list(range(len(tokens)))}],
                      "end": [rid]})
    return steps


def tail_one_by_one(requests: dict[str, list[int]], tail: int = 32) -> list[dict]:
    """Most of the request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, tokens in requests.items():
        head = max(len(tokens) - tail, 1)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": tokens[:head], "want": list(range(head))}],
                      "end": []})
        for i in range(head, len(tokens)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [tokens[i]], "want": [0]}],
                          "end": [rid] if i == len(tokens) - 1 else []})
        if head == len(tokens):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests: dict[str, list[int]], sizes=(7, 2, 16, 3, 2, 5, 33, 2, 9, 17)) -> list[dict]:
    """Portions of changing size, down to two tokens, crossing pages at odd offsets."""
    steps = []
    for rid, tokens in requests.items():
        fed = 0
        turn = 0
        while fed < len(tokens):
            size = min(sizes[turn % len(sizes)], len(tokens) - fed)
            if len(tokens) - fed - size == 1:  # never leave a one-token rest: portions have two tokens or more
                size += 1
            turn += 1
            chunk = tokens[fed:fed + size]
            fed += size
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": chunk, "want": list(range(size))}],
                          "end": [rid] if fed == len(tokens) else []})
    return steps


def mixed(requests: dict[str, list[int]], live: int = 4, chunk_sizes=(5, 12, 2, 9, 3), decode_tail: int = 6,
          seed: int = 0) -> list[dict]:
    """Up to ``live`` requests at a time; each step holds portions of some beside
    single tokens of others; a finished request's pages go back and the next
    waiting request starts, so pages are used again."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    active: list[list] = []  # [rid, tokens, fed]
    steps = []
    turn = 0
    while waiting or active:
        while waiting and len(active) < live:
            rid, tokens = waiting.pop(0)
            active.append([rid, tokens, 0])
        entries = []
        ended = []
        for state in active:
            rid, tokens, fed = state
            if rng.random() < 0.25 and len(active) > 1 and len(entries) > 0:
                continue  # this request sits the step out
            left = len(tokens) - fed
            if left <= decode_tail:
                size = 1
            else:
                size = min(chunk_sizes[turn % len(chunk_sizes)], left - decode_tail)
                size = max(size, 1)
            turn += 1
            chunk = tokens[fed:fed + size]
            state[2] = fed + size
            entries.append({"id": rid, "tokens": chunk, "want": list(range(size))})
            if state[2] == len(tokens):
                ended.append(rid)
        active = [s for s in active if s[2] < len(s[1])]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def fixed_portions(requests: dict[str, list[int]], portion: int = 8, live: int = 3, decode_tail: int = 12) -> list[dict]:
    """As a scheduler cuts them: every prompt in portions of one size (its rest last), the last
    ``decode_tail`` tokens one by one, up to ``live`` requests side by side; logits are wanted where a
    sampler would look, at the last token of every portion and at every single token.  The same shapes
    of steps come again and again."""
    waiting = list(requests.items())
    active: list[list] = []
    steps = []
    while waiting or active:
        if waiting and len(active) < live:  # (one newcomer per step: prompts start at different steps)
            rid, tokens = waiting.pop(0)
            active.append([rid, tokens, 0])
        entries, ended = [], []
        for state in active:
            rid, tokens, fed = state
            left = len(tokens) - fed
            size = 1 if left <= decode_tail else min(portion, left - decode_tail)
            state[2] = fed + size
            entries.append({"id": rid, "tokens": tokens[fed:fed + size], "want": [size - 1]})
            if state[2] == len(tokens):
                ended.append(rid)
        active = [s for s in active if s[2] < len(s[1])]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def random_trace(rng, lengths: list[int], vocab: int, page: int, live_most: int = 4) -> tuple[dict[str, list[int]], list[dict]]:
    """Requests of the given lengths with random tokens, and steps that feed them in random cuts: up to
    ``live_most`` live at a time, some left out of a step, portions of one token, two tokens, up to a page's
    edge, one past it, or anything; logits wanted at random places.  ``rng`` is a ``random.Random``."""
    requests = {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}
    waiting, live, steps = list(requests), {}, []
    while waiting or live:
        while waiting and len(live) < live_most and (not live or rng.random() < 0.5):
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for rid in [rid for rid in live if rng.random() < 0.8] or [next(iter(live))]:
            left = len(requests[rid]) - live[rid]
            to_edge = page - live[rid] % page
            kind = rng.random()
            size = (1 if kind < 0.35 else 2 if kind < 0.55 else to_edge if kind < 0.7 else to_edge + 1 if kind < 0.8
                    else rng.randint(1, left))
            size = max(1, min(size, left))
            want = set(rng.sample(range(size), k=min(size, rng.choice([0, 1, 1, 2, size]))))
            if rng.random() < 0.5:
                want.add(size - 1)
            entries.append({"id": rid, "tokens": requests[rid][live[rid]: live[rid] + size], "want": sorted(want)})
            live[rid] += size
            if live[rid] == len(requests[rid]):
                end.append(rid)
        for rid in end:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return requests, steps


def max_live_tokens(steps: list[dict], page: int = 64) -> int:
    """Most tokens live requests hold at any time, each rounded up to ``page``."""
    held: dict[str, int] = {}
    peak = 0
    for step in steps:
        for entry in step["entries"]:
            held[entry["id"]] = held.get(entry["id"], 0) + len(entry["tokens"])
        peak = max(peak, sum(-(-n // page) * page for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return peak


def drive_runner(runner, steps: list[dict]) -> dict[int, np.ndarray]:
    """What bin/trace_run does, in-process."""
    from cie_amd.engine.runner import StepEntry

    out = {}
    for step in steps:
        entries = []
        for item in step["entries"]:
            if not runner.cache.has(item["id"]):
                runner.cache.admit(item["id"])
            entries.append(StepEntry(item["id"], item["tokens"], runner.cache.length(item["id"]), item["want"]))
        if entries:
            logits = runner.run(entries)
            if logits.shape[0]:
                out[step["step"]] = logits.float().cpu().numpy()
        for rid in step["end"]:
            runner.cache.release(rid)
        runner.cache.assert_invariants()
    return out


def by_position(steps: list[dict], outputs: dict[int, np.ndarray]) -> dict[str, dict[int, np.ndarray]]:
    """{request: {position: logits row}} from the per-step arrays."""
    fed: dict[str, int] = {}
    rows: dict[str, dict[int, np.ndarray]] = {}
    for step in steps:
        data = outputs.get(step["step"])
        cursor = 0
        for entry in step["entries"]:
            base = fed.get(entry["id"], 0)
            for place in entry["want"]:
                rows.setdefault(entry["id"], {})[base + place] = data[cursor]
                cursor += 1
            fed[entry["id"]] = base + len(entry["tokens"])
        if data is not None:
            assert cursor == data.shape[0], "logits rows and wanted places disagree"
    return rows


def compare(rows: dict[str, dict[int, np.ndarray]], plain: dict[str, torch.Tensor], rtol: float, atol: float,
            every_position: bool = True) -> float:
    """Assert every position of every request (or, with ``every_position=False``, the
    positions that were asked for) against the plain logits; returns the worst abs difference."""
    worst = 0.0
    for rid, expected in plain.items():
        got = rows[rid]
        if every_position:
            assert sorted(got) == list(range(expected.shape[0])), f"{rid}: positions {sorted(got)[:5]}..."
        positions = sorted(got)
        assert positions, f"{rid}: no logits"
        stacked = np.stack([got[p] for p in positions])
        want = expected.numpy()[positions]
        diff = np.abs(stacked - want)
        worst = max(worst, float(diff.max()))
        bad = diff > atol + rtol * np.abs(want)
        if bad.any():
            pos = positions[int(np.argwhere(bad.any(axis=1))[0][0])]
            raise AssertionError(
                f"request {rid}: first wrong position {pos} of {expected.shape[0]}, "
                f"max |diff| there {diff[positions.index(pos)].max():.3e}, overall {diff.max():.3e}"
            )
    return worst


def closer_than_plain_bfloat16(rows: dict[str, dict[int, np.ndarray]], plain: dict[str, torch.Tensor],
                               rough: dict[str, torch.Tensor]) -> tuple[float, float, float, float]:
    """What bfloat16 costs at a model's widths is measured, not assumed: ``rough`` are the logits of the plain
    implementation run in bfloat16 throughout, ``plain`` those in float32.  The engine (float32 residual
    stream, softmax and sums) has to be closer to the float32 logits than that: root mean square no larger,
    worst difference at most 1.5 times.  Returns (rms, worst, plain rms, plain worst)."""
    def errors(logits_of):
        square, count, worst = 0.0, 0, 0.0
        for rid, by_pos in rows.items():
            for pos in by_pos:
                diff = logits_of(rid, pos) - plain[rid][pos]
                square += float((diff ** 2).sum())
                count += diff.numel()
                worst = max(worst, float(diff.abs().max()))
        return (square / count) ** 0.5, worst

    plain_rms, plain_worst = errors(lambda rid, pos: rough[rid][pos].float())
    rms, worst = errors(lambda rid, pos: torch.from_numpy(rows[rid][pos]))
    assert rms <= plain_rms and worst <= 1.5 * plain_worst, (rms, worst, plain_rms, plain_worst)
    return rms, worst, plain_rms, plain_worst


def greedy_tokens_follow_plain(plain_forward, prompt: list[int], got: list[int], rough_forward=None,
                               floor: float = 1e-4) -> int:
    """Every generated token against the plain model, teacher-forced on what was generated: token i must
    be the arg-max of the plain logits after ``prompt + got[:i]``, or, where 16-bit rounding may turn a
    near-tie, lie within twice the distance between the plain logits in float32 and in bfloat16
    (``rough_forward``) of that maximum.  Returns how many tokens were near-ties that went the other way."""
    turned = 0
    for index, token in enumerate(got):
        context = list(prompt) + list(got[:index])
        row = plain_forward(context)[-1].float()
        best = int(row.argmax())
        if token == best:
            continue
        margin = floor
        if rough_forward is not None:
            margin = max(floor, 2.0 * float((rough_forward(context)[-1].float() - row).abs().max()))
        gap = float(row[best] - row[token])
        assert gap <= margin, f"token {index}: got {token} (logit {float(row[token]):.5f}), plain picks {best} " \
                              f"({float(row[best]):.5f}); gap {gap:.2e} exceeds {margin:.2e}"
        turned += 1
    return turned


def drawn_tokens_follow_plain(plain_forward, prompt: list[int], got: list[int], temperature: float,
                              uniforms: list[float], slack: float = 1e-4) -> int:
    """Temperature sampling end to end: token i must be the first index at which the running sum of
    softmax(plain logits / temperature) passes ``uniforms[i]``, or a neighbour of it when the number
    falls within ``slack`` of the boundary between the two.  Returns the boundary cases."""
    close = 0
    for index, (token, u) in enumerate(zip(got, uniforms)):
        row = plain_forward(list(prompt) + list(got[:index]))[-1].double()
        p = torch.softmax(row / temperature, dim=-1)
        cdf = torch.cumsum(p, dim=-1)
        expected = int(torch.searchsorted(cdf, torch.tensor(u, dtype=torch.float64), right=True))
        expected = min(expected, row.numel() - 1)
        if token == expected:
            continue
        low = float(cdf[token - 1]) if token > 0 else 0.0
        assert low - slack <= u < float(cdf[token]) + slack, \
            f"token {index}: got {token} whose share of [0, 1) is [{low:.6f}, {float(cdf[token]):.6f}), the number is {u:.6f}"
        close += 1
    return close

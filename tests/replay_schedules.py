"""Schedules for trace replay: the same requests cut into steps in different
ways.  A schedule is a list of step dicts in the replay tool's input format;
``expected_rows`` lists, per step, the (request, position) of every wanted row."""
import random


def roundup(n, m=64):
    return -(-n // m) * m


def whole(requests):
    """Each request alone and whole, one step each."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks,
                                               "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def tail_decoded(requests, tail=32):
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [
            {"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for p in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": [toks[p]], "want": [0]}],
                "end": [rid] if p == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests, sizes=(23, 9, 16, 5, 3, 2, 2, 31, 2, 7, 1, 17)):
    """Portions of changing size, down to two tokens (and one)."""
    steps = []
    for rid, toks in requests.items():
        pos, i = 0, 0
        while pos < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - pos)
            i += 1
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": toks[pos:pos + n], "want": list(range(n))}],
                "end": [rid] if pos + n == len(toks) else []})
            pos += n
    return steps


def mixed(requests, prompt_lens, max_live=4, seed=0, max_portion=24):
    """Up to ``max_live`` live requests: portions of some beside single tokens
    of others; a request is sometimes left out of a step; finished requests end
    and their pages go to the requests admitted after them.  ``prompt_lens[rid]``
    tokens are fed in portions, the rest one by one."""
    rng = random.Random(seed)
    waiting = list(requests)
    live, done_pos = [], {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid = waiting.pop(0)
            live.append(rid)
            done_pos[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                   # left out of this step
            toks, pos = requests[rid], done_pos[rid]
            if pos < prompt_lens[rid]:
                n = min(rng.choice([2, 3, 5, 8, 13, max_portion]), prompt_lens[rid] - pos)
            else:
                n = 1
            n = min(n, len(toks) - pos)
            want = list(range(n)) if n <= 3 or rng.random() < 0.7 else [0, n - 1]
            entries.append({"id": rid, "tokens": toks[pos:pos + n], "want": want})
            done_pos[rid] = pos + n
            if pos + n == len(toks):
                ended.append(rid)
                live.remove(rid)
        if not entries:
            continue
        rng.shuffle(entries)
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def max_tokens_needed(steps, m=64):
    """Largest sum over live requests of their length rounded up to ``m``,
    taken while a step runs (before its ``end`` applies)."""
    held, peak = {}, 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(roundup(n, m) for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return peak


def expected_rows(steps):
    """{step: [(request, absolute position), ...]} in output order."""
    pos, out = {}, {}
    for st in steps:
        rows = []
        for e in st["entries"]:
            start = pos.get(e["id"], 0)
            rows += [(e["id"], start + w) for w in e["want"]]
            pos[e["id"]] = start + len(e["tokens"])
        for rid in st["end"]:
            pos.pop(rid, None)
        if rows:
            out[st["step"]] = rows
    return out

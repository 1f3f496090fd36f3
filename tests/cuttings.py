"""Ways of cutting the same requests into steps, in the trace format of
bin/trace_run: a list of {"step", "entries": [{"id", "tokens", "want"}], "end"}.
Every token's logits are wanted, so that all cuttings can be compared place by
place."""
import random


def _entry(rid, tokens, lo, hi):
    return {"id": rid, "tokens": list(tokens[lo:hi]), "want": list(range(hi - lo))}


def whole(seqs):
    """Each request alone and whole: one step per request."""
    return [{"step": i, "entries": [_entry(rid, toks, 0, len(toks))], "end": [rid]}
            for i, (rid, toks) in enumerate(seqs.items())]


def tail_decode(seqs, tail=32):
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in seqs.items():
        n = len(toks)
        head = max(1, n - tail)
        cuts = [(0, head)] + [(i, i + 1) for i in range(head, n)]
        for j, (lo, hi) in enumerate(cuts):
            steps.append({"step": len(steps), "entries": [_entry(rid, toks, lo, hi)],
                          "end": [rid] if j == len(cuts) - 1 else []})
    return steps


def portions(seqs, sizes=(7, 2, 13, 2, 5, 3, 17, 2, 1, 4)):
    """One request at a time in portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in seqs.items():
        lo, k = 0, 0
        while lo < len(toks):
            hi = min(len(toks), lo + sizes[k % len(sizes)])
            k += 1
            steps.append({"step": len(steps), "entries": [_entry(rid, toks, lo, hi)],
                          "end": [rid] if hi == len(toks) else []})
            lo = hi
    return steps


def mixed(seqs, seed=0, max_live=4, prompt_frac=0.6):
    """Up to ``max_live`` live requests: the first part of each goes in portions
    of random size (sometimes skipping a step), the rest token by token, all in
    shared steps; a request that ends makes room for the next, whose pages are
    the ones just given back."""
    rng = random.Random(seed)
    waiting = list(seqs.items())
    live = {}          # rid -> [tokens, done, prompt_len]
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0, max(2, int(len(toks) * prompt_frac))]
        entries, ended = [], []
        for rid in list(live):
            toks, done, plen = live[rid]
            if len(live) > 1 and rng.random() < 0.15:
                continue                      # left out of this step, goes on later
            if done < plen:
                n = min(plen - done, rng.choice([2, 3, 5, 8, 16, 24, 33]))
            else:
                n = 1
            entries.append(_entry(rid, toks, done, done + n))
            live[rid][1] = done + n
            if done + n == len(toks):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def max_live_tokens(steps, round_to=64):
    """The --max-tokens a trace needs: the most tokens live requests hold at any
    time, each request's count rounded up to a multiple of ``round_to``."""
    held, peak = {}, 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return peak


def decoders_beside_a_portion(shorts, long_id, long_tokens, tails, portion=24, per_step=8,
                              want_prompt_rows="all"):
    """Many requests that decode together beside one prompt that arrives in portions.

    ``shorts``: {request: tokens}; request r decodes its last ``tails[r]`` tokens one by one
    (the others before them go in as one entry, ``per_step`` requests a step). Then every step
    brings one token of every short request that still has some, and a portion of ``long_id``
    while it lasts; with different tails the number of decoding rows falls from step to step.
    ``want_prompt_rows``: "all" rows of the prompt entries or only their "last"."""
    def prompt_entry(rid, toks, lo, hi):
        e = _entry(rid, toks, lo, hi)
        if want_prompt_rows == "last":
            e["want"] = [hi - lo - 1]
        return e

    steps = []
    ids = list(shorts)
    for i in range(0, len(ids), per_step):
        steps.append({"step": len(steps), "end": [], "entries": [
            prompt_entry(r, shorts[r], 0, len(shorts[r]) - tails[r]) for r in ids[i:i + per_step]]})
    done_long, s = 0, 0
    while done_long < len(long_tokens) or any(s < tails[r] for r in ids):
        entries, ended = [], []
        for r in ids:
            if s < tails[r]:
                at = len(shorts[r]) - tails[r] + s
                entries.append(_entry(r, shorts[r], at, at + 1))
                if s == tails[r] - 1:
                    ended.append(r)
        if done_long < len(long_tokens):
            hi = min(len(long_tokens), done_long + portion)
            entries.append(prompt_entry(long_id, long_tokens, done_long, hi))
            done_long = hi
            if hi == len(long_tokens):
                ended.append(long_id)
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        s += 1
    return steps


def wanted_places(steps):
    """{request: sorted positions whose logits the steps ask for}."""
    fed, out = {}, {}
    for st in steps:
        for e in st["entries"]:
            base = fed.get(e["id"], 0)
            out.setdefault(e["id"], []).extend(base + w for w in e["want"])
            fed[e["id"]] = base + len(e["tokens"])
    return {r: sorted(p) for r, p in out.items()}

"""Ways of cutting the same requests into trace steps, and putting the answers back together.

A request is a fixed list of token ids; a plan is a list of trace steps (the JSON objects that
bin/trace_run reads).  Every plan asks for the logits at every position of every request, so the
results of all plans can be compared with the plain implementation's whole-sequence logits.
"""
import numpy as np


def whole(requests):
    """Each request alone and whole: one step per request."""
    return [{"step": i, "entries": [{"id": rid, "tokens": list(toks), "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def tail_one_by_one(requests, tail=32):
    """Each request alone: all but the last `tail` tokens in one step, then the rest one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": list(toks[:head]),
                                                       "want": list(range(head))}], "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    return steps


def unequal_batches(batches):
    """`batches`: a list of {id: (tokens, prompt_len)}.  The requests of a batch start together with
    their prompts in one step, then go on by one token each; a request ends when its tokens are used
    up, the others go on.  The next batch starts when the one before has ended."""
    steps = []
    for batch in batches:
        fed = {rid: p for rid, (toks, p) in batch.items()}
        entries = [{"id": rid, "tokens": list(toks[:p]), "want": list(range(p))} for rid, (toks, p) in batch.items()]
        ended = [rid for rid, (toks, p) in batch.items() if p == len(toks)]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        live = [rid for rid in batch if rid not in ended]
        while live:
            entries = [{"id": rid, "tokens": [batch[rid][0][fed[rid]]], "want": [0]} for rid in live]
            for rid in live:
                fed[rid] += 1
            ended = [rid for rid in live if fed[rid] == len(batch[rid][0])]
            steps.append({"step": len(steps), "entries": entries, "end": ended})
            live = [rid for rid in live if rid not in ended]
    return steps


def max_live_tokens(steps):
    """What --max-tokens has to be for a plan: the most tokens live requests hold at any time, each
    request's count rounded up to a multiple of 64."""
    held, worst = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // 64) * 64 for n in held.values()))
        for rid in s["end"]:
            held.pop(rid)
    return worst


def collect(steps, logits_of_step, vocab):
    """{request id: [len, vocab] array} from the per-step outputs (`logits_of_step(step) -> [wanted, vocab]`)."""
    rows, seen = {}, {}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        out = np.asarray(logits_of_step(s["step"]), dtype=np.float32).reshape(-1, vocab) if wanted else None
        assert out is None or out.shape[0] == wanted, f"step {s['step']}: {out.shape[0]} rows for {wanted} places"
        r = 0
        for e in s["entries"]:
            base = seen.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[base + w] = out[r]
                r += 1
            seen[e["id"]] = base + len(e["tokens"])
    return {rid: np.stack([by_pos[i] for i in sorted(by_pos)]) for rid, by_pos in rows.items()}

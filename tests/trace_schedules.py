"""Schedules that replay the same requests in different ways (records for bin/trace_run)."""


def whole(requests):
    """Each request alone and whole; every position wanted."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps


def last_one_by_one(requests, tail=32):
    """The first len - tail tokens in one step, the last `tail` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for j in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[j]], "want": [0]}],
                          "end": [rid] if j == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def batches(requests, batch_size, prefill_fraction=0.5):
    """Batches of unequal lengths, one after another: each batch starts together with a prompt part of
    every request, then goes on by one token each; shorter requests end earlier."""
    steps = []
    ids = list(requests)
    for b in range(0, len(ids), batch_size):
        group = ids[b:b + batch_size]
        done = {}
        entries = []
        for rid in group:
            n = max(1, int(len(requests[rid]) * prefill_fraction))
            done[rid] = n
            entries.append({"id": rid, "tokens": requests[rid][:n], "want": list(range(n))})
        ends = [rid for rid in group if done[rid] == len(requests[rid])]
        steps.append({"step": len(steps), "entries": entries, "end": ends})
        live = [rid for rid in group if rid not in ends]
        while live:
            entries, ends = [], []
            for rid in live:
                entries.append({"id": rid, "tokens": [requests[rid][done[rid]]], "want": [0]})
                done[rid] += 1
                if done[rid] == len(requests[rid]):
                    ends.append(rid)
            steps.append({"step": len(steps), "entries": entries, "end": ends})
            live = [rid for rid in live if rid not in ends]
    return steps


def chunked(requests, sizes):
    """Each request alone, fed in portions whose sizes cycle through `sizes`; every position wanted."""
    steps = []
    for rid, toks in requests.items():
        at, turn = 0, 0
        while at < len(toks):
            n = min(sizes[turn % len(sizes)], len(toks) - at)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
                          "end": [rid] if at + n == len(toks) else []})
            at += n
            turn += 1
    return steps


def joining(requests, every=2, burst=4):
    """Requests join a batch that is running: every `every` steps the next request starts with half of its tokens in
    one portion, while those already running go on by one token, or by `burst` tokens now and then; a request
    leaves when its tokens run out."""
    steps = []
    waiting = list(requests)
    done, live = {}, []
    while waiting or live:
        k = len(steps)
        entries = []
        for i, rid in enumerate(live):
            n = burst if (k + i) % 4 == 0 else 1
            n = min(n, len(requests[rid]) - done[rid])
            entries.append({"id": rid, "tokens": requests[rid][done[rid]:done[rid] + n], "want": list(range(n))})
            done[rid] += n
        if waiting and (k % every == 0 or not live):
            rid = waiting.pop(0)
            n = max(1, (len(requests[rid]) + 1) // 2)
            entries.append({"id": rid, "tokens": requests[rid][:n], "want": list(range(n))})
            done[rid] = n
            live.append(rid)
        ends = [rid for rid in live if done[rid] == len(requests[rid])]
        steps.append({"step": k, "entries": entries, "end": ends})
        live = [rid for rid in live if rid not in ends]
    return steps


def collect(steps, outputs, vocab):
    """outputs: {step: array [wanted, vocab]} -> {request id: array [len, vocab]} in position order."""
    import numpy as np
    rows = {}
    for rec in steps:
        if rec["step"] not in outputs:
            continue
        arr = outputs[rec["step"]].reshape(-1, vocab)
        o = 0
        for e in rec["entries"]:
            for _ in e.get("want", []):
                rows.setdefault(e["id"], []).append(arr[o])
                o += 1
        assert o == arr.shape[0]
    return {rid: np.stack(v) for rid, v in rows.items()}


def held_tokens(steps, page=64):
    """The most tokens live requests hold at any time, each rounded up to a page."""
    held, most = {}, 0
    for rec in steps:
        for e in rec["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(-(-n // page) * page for n in held.values()))
        for rid in rec["end"]:
            del held[rid]
    return most


def run_on_model(model, cache, steps):
    """The schedule's steps through model.step on `cache` (any page size); {step: logits [wanted, vocab]} as arrays."""
    slot_of, out = {}, {}
    for rec in steps:
        slots, counts, flat, want, offset = [], [], [], [], 0
        for e in rec["entries"]:
            if e["id"] not in slot_of:
                slot_of[e["id"]] = cache.acquire()
            slots.append(slot_of[e["id"]])
            counts.append(len(e["tokens"]))
            flat.extend(e["tokens"])
            want.extend(offset + w for w in e.get("want", []))
            offset += len(e["tokens"])
        logits = model.step(cache, slots, flat, counts=counts, want=want)
        if logits is not None:
            out[rec["step"]] = logits.float().cpu().numpy()
        for rid in rec["end"]:
            cache.release(slot_of.pop(rid))
    assert not slot_of
    return out

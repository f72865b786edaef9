"""A slow sampler oracle in double precision, written from the reference's rules with plain loops.

Rules (paths relative to the reference's root): candidates are finite logits sorted descending with
ties by lower index; weight exp(l/t - l_max/t); normalise (crates/leone/src/sampler.rs:502-534).
Stages in order, each on the renormalised result of the one before, each keeping at least one
(crates/leone/src/sampler.rs:559-606): top-k keeps k; top-p the shortest prefix whose mass reaches p;
min-p those >= p * highest.  The token is the first in id order with u < cumulative probability, else
the last eligible (crates/leone/src/sampler.rs:843-858).  The uniform value comes from
splitmix64(seed ^ splitmix64(position ^ purpose)) >> 11, times 2^-53 (crates/leone/src/sampler.rs:84-95, 166-171).
"""
import math

M = (1 << 64) - 1
SELECT = 0xBF58476D1CE4E5B9


def mix(v):
    z = (v + 0x9E3779B97F4A7C15) & M
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
    return z ^ (z >> 31)


def uniform(seed, position):
    return (mix((seed & M) ^ mix((position & M) ^ SELECT)) >> 11) / float(1 << 53)


def greedy(logits):
    best = None
    for i, v in enumerate(logits):
        v = float(v)
        if math.isnan(v) or math.isinf(v):
            continue
        if best is None or v > best[1]:
            best = (i, v)
    return -1 if best is None else best[0]


def distribution(logits, temperature, stages=()):
    cands = [(float(v), i) for i, v in enumerate(logits) if not (math.isnan(float(v)) or math.isinf(float(v)))]
    if not cands:
        raise ValueError("no finite logit")
    cands.sort(key=lambda c: (-c[0], c[1]))
    top = cands[0][0] / temperature
    weights = [math.exp(v / temperature - top) for v, _ in cands]
    total = math.fsum(weights)
    probs = [w / total for w in weights]
    for name, value in stages:
        if name == "top_k":
            keep = min(int(value), len(probs))
        elif name == "top_p":
            keep, mass = len(probs), 0.0
            for n, p in enumerate(probs):
                mass += p
                if mass >= value:
                    keep = n + 1
                    break
        elif name == "min_p":
            keep = 0
            while keep < len(probs) and probs[keep] >= value * probs[0]:
                keep += 1
        else:
            raise ValueError(name)
        keep = max(1, keep)
        probs = probs[:keep]
        cands = cands[:keep]
        total = math.fsum(probs)
        probs = [p / total for p in probs]
    out = [0.0] * len(logits)
    for (_, i), p in zip(cands, probs):
        out[i] = p
    return out


def select(probs, u):
    running, last = 0.0, None
    for i, p in enumerate(probs):
        if p <= 0.0:
            continue
        last = i
        running += p
        if u < running:
            return i
    return last


def dry(logits, history, multiplier, base, allowed, window, breakers=()):
    """The repeated-suffix penalty, by comparing suffixes outright: for every earlier position
    holding the last token, the longest common run ending there and at the end, cut where a
    breaker would be crossed; a run of at least ``allowed`` costs multiplier * base^(run - allowed)
    on the token after the earlier position (crates/leone/src/penalty.rs:198-249)."""
    out = [float(v) for v in logits]
    recent = list(history)[-window:] if window > 0 else []
    if multiplier <= 0 or len(recent) < 2:
        return out
    end = len(recent) - 1
    best = {}
    for at in range(end):
        run = 0
        while run <= at and recent[at - run] == recent[end - run] and (run == 0 or recent[end - run] not in breakers):
            run += 1
        if run == 0 or run < allowed:
            continue
        follower = recent[at + 1]
        if follower in breakers:
            continue
        cost = multiplier
        for _ in range(run - allowed):
            cost *= base
        best[follower] = max(best.get(follower, 0.0), cost)
    for token, cost in best.items():
        if token < len(out):
            out[token] -= cost
    return out


def mirostat(probs, bound, target, rate, u):
    """One Mirostat v2 draw: (token, new bound) (crates/leone/src/sampler.rs:398-446)."""
    kept = [p if p > 0.0 and -math.log(p) <= bound else 0.0 for p in probs]
    if sum(kept) == 0.0:
        top = max(range(len(probs)), key=lambda i: (probs[i], -i))
        kept[top] = probs[top]
    total = math.fsum(kept)
    token = select([p / total for p in kept], u)
    bound = bound - rate * (-math.log(probs[token]) - target)
    return token, max(bound, 2.0 ** -52)

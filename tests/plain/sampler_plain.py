"""A plain sampler with the reference's order of operations (sampling/Sampler.java:346-456), in float64:
penalties -> bias -> greedy? -> candidates (top-k, else everything) -> weights exp((z - max) / T) -> top-p on the
candidates sorted descending (shortest prefix whose share of the candidates' mass reaches top_p; the crossing token
is kept) -> min-p (weights below min_p of the top token's weight 1 are dropped) -> one draw.

The draw walks the kept tokens in index order with a given uniform number (the engine's choice; the reference walks
them sorted, with its own random stream: same distribution). Tokens whose logit equals a threshold are all kept.
"""
import math
from typing import Dict, Iterable, List, Optional, Sequence


def apply_penalties(logits: List[float], seen: Iterable[int], generated: Dict[int, int], rep: float, pres: float,
                    freq: float, bias: Optional[Dict[int, float]] = None) -> List[float]:
    """Sampler.java:434-456: z = z > 0 ? z / rep : z * rep for every token seen in prompt or output; then
    z -= presence + frequency * count for generated ones; then the bias."""
    z = list(logits)
    for t in set(seen) | set(generated):
        if rep != 1:
            z[t] = z[t] / rep if z[t] > 0 else z[t] * rep
        c = generated.get(t, 0)
        if c > 0:
            z[t] -= pres + freq * c
    for t, b in (bias or {}).items():
        z[t] += b
    return z


def argmax(z: Sequence[float]) -> int:
    """Sampler.java:458-466: a `>` scan from 0, so the lowest index among equal maxima."""
    best = 0
    for i in range(1, len(z)):
        if z[i] > z[best]:
            best = i
    return best


def kept_weights(z: Sequence[float], temperature: float, top_k: int, top_p: float, min_p: float) -> Dict[int, float]:
    """token -> unnormalised weight of every token that can be drawn (Sampler.java:360-411)."""
    V = len(z)
    inv_t = 1.0 / temperature
    order = sorted(range(V), key=lambda i: (-z[i], i))
    if 0 < top_k < V:
        kth = z[order[top_k - 1]]
        cand = [i for i in order if z[i] >= kth]  # ties with the k-th are all kept
    else:
        cand = order
    zmax = z[cand[0]]
    w = {i: math.exp((z[i] - zmax) * inv_t) for i in cand}
    total = sum(w.values())
    kept = list(cand)
    if top_p < 1.0:
        cum = 0.0
        cut = len(cand)
        for n, i in enumerate(cand):
            cum += w[i] / total
            if cum >= top_p:
                cut = n + 1
                break
        edge = z[cand[cut - 1]]
        kept = [i for i in cand if z[i] >= edge]
    if min_p > 0:
        kept = [i for i in kept if w[i] >= min_p]
    return {i: w[i] for i in kept}


def draw(weights: Dict[int, float], u: float) -> int:
    """First token, in index order, whose cumulative weight exceeds u * total."""
    total = sum(weights.values())
    r = u * total
    acc = 0.0
    last = None
    for i in sorted(weights):
        acc += weights[i]
        last = i
        if r < acc:
            return i
    return last


def sample(z: Sequence[float], temperature: float, top_k: int, top_p: float, min_p: float, u: float) -> int:
    if temperature == 0 or top_k == 1:
        return argmax(z)
    return draw(kept_weights(z, temperature, top_k, top_p, min_p), u)


def token_logprob(logits: Sequence[float], token: int, top: int):
    """engine/TokenLogprob.java:22-54: logprob(t) = z_t - (max + log(sum_j exp(z_j - max))) of the raw logits, and the
    `top` largest logits with theirs, most likely first; the insertion there moves a new entry only past strictly
    smaller ones, so among equal logits the lower index comes first. Returns (logprob, ids, logprobs)."""
    zmax = max(logits)
    lse = zmax + math.log(sum(math.exp(z - zmax) for z in logits))
    order = sorted(range(len(logits)), key=lambda i: (-logits[i], i))[:top]
    return logits[token] - lse, order, [logits[i] - lse for i in order]

"""Plain sampler written from picolm/sampler.c, in float64, one function a step.

Where sampler.c leaves an order open (qsort on equal probabilities, sampler.c:27-33,:67)
this file fixes it: equal probabilities keep ascending token order.
"""
from __future__ import annotations

import numpy as np

MASK64 = (1 << 64) - 1


def xorshift64(state: int) -> int:
    """sampler.c:10-17. Returns the new state, which is also the output."""
    x = state & MASK64
    x ^= (x << 13) & MASK64
    x ^= x >> 7
    x ^= (x << 17) & MASK64
    return x


def rand_float(state: int) -> tuple[float, int]:
    """sampler.c:19-21: (float)(x >> 11) / (float)(1 << 53), both rounded to float32."""
    x = xorshift64(state)
    r = np.float32(np.float32(x >> 11) / np.float32(2.0 ** 53))
    return float(r), x


def init_state(seed: int) -> int:
    """sampler.c:43: a zero seed becomes 42."""
    seed &= MASK64
    return seed if seed else 42


def argmax_first(logits: np.ndarray) -> int:
    """sampler.c:50-55: strict '>' keeps the first maximum."""
    best = 0
    for i in range(1, len(logits)):
        if logits[i] > logits[best]:
            best = i
    return best


def sample(logits, temperature: float, top_k: int, top_p: float, min_p: float,
           state: int) -> tuple[int, int]:
    """One draw; returns (token, new rng state).  sampler.c:48-125."""
    logits = np.asarray(logits, dtype=np.float64)
    V = len(logits)
    # the options are floats in picolm (sampler.h:6-12): round them as it does
    temperature = float(np.float32(temperature))
    top_p = float(np.float32(top_p))
    min_p = float(np.float32(min_p))
    if temperature <= 0.0:
        return argmax_first(logits), state
    # 1. softmax of the raw logits (:59)
    e = np.exp(logits - np.max(logits))
    p = e / np.sum(e)
    # 2. sort by probability, descending (:62-67)
    order = sorted(range(V), key=lambda i: (-p[i], i))
    ps = np.array([p[i] for i in order])
    # 3. top-k (:70-73)
    k_limit = top_k if 0 < top_k < V else V
    # 4. top-p inside top-k (:76-82)
    cum, cutoff = 0.0, 0
    for i in range(k_limit):
        cum += ps[i]
        cutoff = i + 1
        if cum >= top_p:
            break
    # 5. min-p (:85-95)
    if min_p > 0.0 and cutoff > 1:
        thr = min_p * ps[0]
        new_cutoff = 0
        for i in range(cutoff):
            if ps[i] >= thr:
                new_cutoff = i + 1
        cutoff = max(new_cutoff, 1)
    # 6. temperature on the kept ones, renormalised (:98-109)
    scaled = np.power(ps[:cutoff], 1.0 / temperature)
    total = np.sum(scaled)
    if total > 0:
        scaled = scaled / total
    # 7. draw (:112-121)
    r, state = rand_float(state)
    acc = 0.0
    result = order[0]
    for i in range(cutoff):
        acc += scaled[i]
        if acc > r:
            result = order[i]
            break
    return result, state

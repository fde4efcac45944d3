"""Plain sampling: the reference's processing of logits into a distribution
(src/tokenvault/sampling.py:40-66) and a draw from it.

The reference draws with one global ``torch.Generator`` in batch order
(src/tokenvault/sampling.py:69-88), which ties a request's tokens to its neighbours.  The
engine instead draws ``u`` in [0, 1) from a counter-based generator keyed by
(engine seed, request stream, index of the output token) and takes the first token, in
vocabulary order, whose cumulative probability exceeds ``u``.  Both are written here in
plain Python/torch so the tests can check the engine's tokens.
"""

from __future__ import annotations

import torch

MASK64 = (1 << 64) - 1


def splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & MASK64
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & MASK64
    return x ^ (x >> 31)


def uniform(seed: int, stream: int, counter: int) -> float:
    """24 random bits as a float in [0, 1): exact in fp32."""
    x = splitmix64(seed & MASK64)
    x = splitmix64(x ^ (stream & MASK64))
    x = splitmix64(x ^ (counter & MASK64))
    return (x >> 40) / float(1 << 24)


def processed_probs(logits: torch.Tensor, temperature: float, top_k: int = 0,
                    top_p: float = 1.0) -> torch.Tensor:
    """src/tokenvault/sampling.py:40-66 for one row.  The reference leaves the order of equal
    values to ``torch.sort``; here equal values are kept or dropped together: top-k keeps every
    value >= the k-th largest, top-p keeps a value iff the mass (within the top-k set) of the
    strictly larger values is below ``top_p``."""
    logits = logits.double()
    vocab = logits.shape[-1]
    if temperature == 0.0:
        out = torch.zeros(vocab, dtype=torch.float64)
        out[int(logits.argmax())] = 1.0
        return out
    # the engine multiplies by the fp32 reciprocal of the temperature
    scaled = (logits.float() * (torch.tensor(1.0, dtype=torch.float32) / temperature)).double()
    keep = torch.ones(vocab, dtype=torch.bool)
    if 0 < top_k < vocab:
        kth = torch.sort(scaled, descending=True).values[top_k - 1]
        keep &= scaled >= kth
    if top_p < 1.0:
        probs_k = torch.softmax(scaled.masked_fill(~keep, float("-inf")), -1)
        sv, order = torch.sort(scaled, descending=True, stable=True)
        sp = probs_k[order]
        cum_before = sp.cumsum(-1) - sp
        first = torch.searchsorted(-sv, -sv, right=False)      # first place of each value
        mass_gt = torch.empty(vocab, dtype=torch.float64)
        mass_gt[order] = cum_before[first]
        keep &= mass_gt < top_p
    return torch.softmax(scaled.masked_fill(~keep, float("-inf")), -1)


def draw(probs: torch.Tensor, u: float) -> int:
    """First index whose cumulative probability exceeds ``u``."""
    cdf = probs.double().cumsum(-1)
    idx = int(torch.searchsorted(cdf, torch.tensor(u * float(cdf[-1]), dtype=torch.float64),
                                 right=True))
    return min(idx, probs.shape[-1] - 1)


def draw_margin(probs: torch.Tensor, u: float, token: int) -> float:
    """How far ``u`` lies outside ``token``'s interval of the CDF (0 when inside)."""
    cdf = probs.double().cumsum(-1)
    total = float(cdf[-1])
    lo = float(cdf[token - 1]) / total if token > 0 else 0.0
    hi = float(cdf[token]) / total
    if lo <= u < hi:
        return 0.0
    return min(abs(u - lo), abs(u - hi))

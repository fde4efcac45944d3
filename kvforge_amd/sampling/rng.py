"""Counter-based uniform numbers: ``u = uniform(engine seed, request stream, output index)``.

The reference draws every row of a batch from one ``torch.Generator``
(src/tokenvault/sampling.py:76-88), so a request's tokens depend on its neighbours.  Keying the
draw by request and output index makes sampled tokens independent of batching and chunking.
"""

from __future__ import annotations

_M = (1 << 64) - 1


def _mix(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _M
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _M
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _M
    return x ^ (x >> 31)


def uniform(seed: int, stream: int, counter: int) -> float:
    """24 random bits in [0, 1), exactly representable in fp32."""
    x = _mix(seed & _M)
    x = _mix(x ^ (stream & _M))
    x = _mix(x ^ (counter & _M))
    return (x >> 40) / 16777216.0

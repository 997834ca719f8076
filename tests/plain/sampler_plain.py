"""Plain temperature sampling, written from the engine's stated rule and sharing no code with it:

  u(seed, index) = the top 24 bits of splitmix64's finaliser applied to
                   seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xD1B54A32D192ED03   (mod 2^64), as a fraction of 2^24;
  token          = the first id, in ascending order, at which the cumulative sum of
                   softmax(logits / temperature) exceeds u;   temperature 0: the lowest id among the maxima
                   (the reference's greedy choice, src/engine/model_runner.cpp:131).

Everything here is float64 / numpy uint64."""
import numpy as np


def uniform(seed: int, index: int) -> float:
    with np.errstate(over="ignore"):
        x = np.uint64(seed % (1 << 64)) * np.uint64(0x9E3779B97F4A7C15) + np.uint64(index + 1) * np.uint64(0xD1B54A32D192ED03)
        x ^= x >> np.uint64(30)
        x *= np.uint64(0xBF58476D1CE4E5B9)
        x ^= x >> np.uint64(27)
        x *= np.uint64(0x94D049BB133111EB)
        x ^= x >> np.uint64(31)
    return float(int(x) >> 40) / 16777216.0


def choose(logits, temperature: float, u: float):
    """(token, margin): margin = distance of u from the nearest edge of the chosen token's interval of the cumulative
    distribution (a choice with a tiny margin may fall either way under float32 rounding)."""
    x = np.asarray(logits, dtype=np.float64)
    if temperature == 0.0:
        return int(np.argmax(x)), 1.0
    z = (x - x.max()) / temperature
    p = np.exp(z)
    cdf = np.cumsum(p / p.sum())
    tok = int(np.searchsorted(cdf, u, side="right"))
    tok = min(tok, len(cdf) - 1)
    lo = cdf[tok - 1] if tok else 0.0
    return tok, float(min(u - lo, cdf[tok] - u))

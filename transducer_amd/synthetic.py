"""Seeded synthetic RNN-T loss inputs with the shapes and length distributions of the
benchmark configurations (emissions [B,T,V], predictions [B,U+1,V], labels [B,U] in [1,V),
ragged or full lengths).  numpy's counter-based Philox generator is used so a (config, seed)
pair names one input set wherever the same numpy runs; nothing here touches a GPU."""
from collections import namedtuple

import numpy as np

Config = namedtuple("Config", "name B T U V sigma ragged_T ragged_U")

# U is the longest label; predictions carry U+1 rows.  ragged_* = (low, high) inclusive bounds
# of the uniform length draw, None = every utterance at full length.
CONFIGS = {
    "cfg1": Config("cfg1", 4, 50, 10, 32, 1.0, (25, 50), (1, 10)),
    "cfg2": Config("cfg2", 8, 2000, 100, 100, 1.0, None, None),
    "cfg3a": Config("cfg3a", 8, 2000, 100, 1000, 2.0, (1000, 2000), (50, 100)),
    "cfg3b": Config("cfg3b", 8, 2000, 100, 2000, 2.0, (1000, 2000), (50, 100)),
    "cfg4": Config("cfg4", 32, 2000, 100, 10000, 1.0, (1500, 2000), (75, 100)),
    "cfg5": Config("cfg5", 32, 2000, 100, 10000, 1.0, (1500, 2000), (75, 100)),
}


def lengths(cfg, rng):
    """One utterance is pinned at full T and one at full U when lengths are ragged."""
    B = cfg.B
    if cfg.ragged_T is None:
        il = np.full(B, cfg.T, np.int32)
    else:
        il = rng.integers(cfg.ragged_T[0], cfg.ragged_T[1] + 1, B).astype(np.int32)
        il[0] = cfg.T
    if cfg.ragged_U is None:
        ll = np.full(B, cfg.U, np.int32)
    else:
        ll = rng.integers(cfg.ragged_U[0], cfg.ragged_U[1] + 1, B).astype(np.int32)
        ll[B - 1] = cfg.U
    return il, ll


def make_inputs(cfg, seed=0, near_ties=False, scale=None):
    """-> dict(emissions, predictions, labels, input_lengths, label_lengths) of numpy arrays.

    near_ties: copy 10% of the (t, v) emission entries from another v of the same frame, so
    distinct labels score exactly alike and competing viterbi paths land within rounding."""
    if isinstance(cfg, str):
        cfg = CONFIGS[cfg]
    rng = np.random.Generator(np.random.Philox(key=seed))
    sigma = cfg.sigma if scale is None else scale
    E = rng.standard_normal((cfg.B, cfg.T, cfg.V), dtype=np.float32)
    P = rng.standard_normal((cfg.B, cfg.U + 1, cfg.V), dtype=np.float32)
    if sigma != 1.0:
        E *= np.float32(sigma)
        P *= np.float32(sigma)
    labels = rng.integers(1, cfg.V, (cfg.B, cfg.U)).astype(np.int32)
    il, ll = lengths(cfg, rng)
    if near_ties:
        n = cfg.B * cfg.T * cfg.V
        k = n // 10
        flat = E.reshape(cfg.B * cfg.T, cfg.V)
        rows = rng.integers(0, cfg.B * cfg.T, k)
        dst = rng.integers(1, cfg.V, k)
        src = rng.integers(1, cfg.V, k)
        flat[rows, dst] = flat[rows, src]
    return dict(emissions=E, predictions=P, labels=labels, input_lengths=il, label_lengths=ll)


def small_config(B, T, U, V, sigma=1.0, ragged=True, name="custom"):
    return Config(name, B, T, U, V, sigma, (max(1, T // 2), T) if ragged else None,
                  (min(1, U), U) if ragged else None)

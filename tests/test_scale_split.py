"""The bf16 kernels' way of applying the scale in launches without mask (sfb_scale_parts) and what it leaves of the
error budget: a numpy model of that loop's arithmetic -- power-of-two part of scale * log2(e) on the bf16 queries,
the rest in fp32 per score, probabilities relative to the first block's row maximum, rounded to bf16 for the P V
product, the row sum over the unrounded values -- against float64 attention with the reference's + 1e-6
(ewops.h:86, 93).  Its error must not grow with the size of the scores; rounding queries * scale * log2(e) to bf16 a
second time, as an earlier form of the loop did, does grow and passes the bf16 tolerance for peaked rows."""
import numpy as np
import pytest

import oracle_lib as orc
from sfb import sfb

TOL_BF16 = 1e-2
LOG2E = 1.4426950408889634


def bf16(x):
    return orc.round_bf16(np.asarray(x, np.float32))


@pytest.mark.parametrize("scale", [0.125, 1.0, 0.01, 1 / np.sqrt(32), 1 / np.sqrt(96), 1 / np.sqrt(128), 3.7, 1e-4])
def test_scale_parts(scale):
    pow2, rest = sfb.scale_parts(scale)
    mant, exponent = np.frexp(np.float32(pow2))
    assert mant == 0.5, "a power of two"
    assert 0.70710678 <= rest < 1.41421357
    want = np.float32(scale) * np.float32(LOG2E)
    assert abs(np.float32(pow2) * np.float32(rest) - want) <= np.spacing(want)
    # exact on bf16 values: the product needs no more mantissa bits than the factor had
    q = bf16(np.random.default_rng(1).standard_normal(4096))
    assert np.array_equal(bf16(q * np.float32(pow2)), q * np.float32(pow2))


def model(qmul, scale, split, nkeys=512, d=64, nq=512, seed=0, bs=64):
    rng = np.random.default_rng(seed)
    Q = bf16(rng.standard_normal((nq, d)) * qmul)
    K = bf16(rng.standard_normal((nkeys, d)))
    V = bf16(rng.standard_normal((nkeys, d)))
    S = Q.astype(np.float64) @ K.astype(np.float64).T
    P = np.exp((S - S.max(1, keepdims=True)) * scale)
    want = (P / (P.sum(1, keepdims=True) + 1e-6)) @ V.astype(np.float64)
    if split:
        pow2, rest = (np.float32(x) for x in sfb.scale_parts(scale))
        queries = Q * pow2
    else:
        queries, rest = bf16(Q * np.float32(scale * LOG2E)), np.float32(1.0)
    scores = (queries.astype(np.float64) @ K.astype(np.float64).T).astype(np.float32)
    offset = scores[:, :bs].max(1, keepdims=True)
    p = np.exp2(((scores - offset) * rest).astype(np.float32)).astype(np.float32)
    assert np.isfinite(p).all() and p.sum(1).max() < 2.0 ** 100, "the loop with the fixed offset is what is modelled"
    out = (bf16(p).astype(np.float64) @ V.astype(np.float64)) / (p.sum(1, keepdims=True, dtype=np.float64) + 1e-6)
    return float(np.abs(out - want).max() / np.abs(want).max())


@pytest.mark.parametrize("qmul,scale", [(1.0, 0.125), (6.0, 0.125), (1.0, 1.0), (10.0, 0.125), (2.0, 1.0)])
def test_error_of_the_split_scale_does_not_grow_with_the_scores(qmul, scale):
    err = max(model(qmul, scale, True, seed=s) for s in range(2))
    assert err <= 0.5 * TOL_BF16, err


def test_a_second_rounding_of_the_queries_would_pass_the_tolerance():
    assert model(1.0, 0.125, False) <= 0.5 * TOL_BF16              # harmless for scores of a few units ...
    assert model(10.0, 0.125, False) > TOL_BF16                    # ... and out of tolerance for peaked rows
    assert model(10.0, 0.125, True) <= 0.5 * TOL_BF16

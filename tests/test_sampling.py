"""The host sampler against exact distributions and the reference's vectors
(crates/engine/src/sampler.rs:278-406)."""
import numpy as np
import pytest

from rust_llm_inference_server_amd.sampling import (Sampler, SamplingParams,
                                                    apply_repetition_penalty, argmax, draw,
                                                    nucleus, row_key)


def test_argmax_ties_go_to_the_lowest_index():
    assert argmax(np.array([0.1, 3.0, -1.0, 3.0], dtype=np.float32)) == 1
    assert argmax(np.array([-np.inf, -5.0], dtype=np.float32)) == 1


def test_repetition_penalty_vector():
    l = np.array([2.0, -2.0, 1.0], dtype=np.float32)
    apply_repetition_penalty(l, [0, 1, 1, 0], 2.0)
    assert l.tolist() == [1.0, -4.0, 1.0]


def test_nucleus_and_draw():
    w = np.array([0.5, 0.3, 0.15, 0.05])
    assert nucleus(w, 1.0, 0.5) == 1 and nucleus(w, 1.0, 0.51) == 2 and nucleus(w, 1.0, 0.95) == 3
    assert nucleus(w[:2], 1.0, 0.9) is None              # all of them together fall short
    assert draw(w, 1.0, 0.0) == 0 and draw(w, 1.0, 0.49) == 0 and draw(w, 1.0, 0.5) == 1
    assert draw(w, 1.0, 0.999) == 3
    assert draw(np.array([0.2, 0.0]), 0.2, 1.0 - 1e-17) == 0        # falls back to the last positive


def test_device_modes():
    assert Sampler(SamplingParams()).device_mode(5) == (0, 0.0)
    s = Sampler(SamplingParams(temperature=0.5, seed=9))
    assert s.device_mode(5) == (row_key(9, 5), 2.0)
    for p in (SamplingParams(temperature=0.5, top_k=5), SamplingParams(temperature=0.5, top_p=0.9),
              SamplingParams(repetition_penalty=1.1)):
        assert Sampler(p).device_mode(5) is None
    assert Sampler(SamplingParams(top_k=5)).device_mode(0) == (0, 0.0)   # greedy ignores top-k


def frequencies(params, logits, n=20000):
    s = Sampler(params)
    counts = np.zeros(len(logits))
    for pos in range(n):
        counts[s.sample(np.array(logits, dtype=np.float32), [], pos)] += 1
    return counts / n


def exact(logits, t, top_k=0, top_p=1.0):
    l = np.array(logits, dtype=np.float64)
    w = np.exp((l - l.max()) / t)
    order = np.lexsort((np.arange(len(l)), -l))
    if top_k:
        order = order[:top_k]
    total = w[order].sum() if top_k else w.sum()
    keep = len(order)
    if top_p < 1.0:
        acc = np.cumsum(w[order] / total)
        keep = int(np.nonzero(acc >= top_p)[0][0]) + 1
    p = np.zeros(len(l))
    p[order[:keep]] = w[order[:keep]] / w[order[:keep]].sum()
    return p


@pytest.mark.parametrize("kw", [dict(), dict(top_k=3), dict(top_p=0.8), dict(top_k=4, top_p=0.7),
                                dict(top_k=1)])
def test_every_mode_follows_the_exact_filtered_softmax(kw):
    logits = [0.0, 1.0, 2.0, -1.0, 1.5, 0.5]
    got = frequencies(SamplingParams(temperature=0.7, seed=7, **kw), logits)
    assert np.abs(got - exact(logits, 0.7, **kw)).max() < 0.015       # sampler.rs tests: 0.015


def test_same_seed_same_tokens_and_temperature_zero_is_greedy():
    logits = np.random.default_rng(0).normal(size=50).astype(np.float32)
    a = Sampler(SamplingParams(temperature=1.0, seed=3))
    b = Sampler(SamplingParams(temperature=1.0, seed=3))
    assert [a.sample(logits, [], p) for p in range(30)] == [b.sample(logits, [], p) for p in range(30)]
    g = Sampler(SamplingParams(temperature=0.0, top_k=5, top_p=0.5))
    assert g.sample(logits, [], 0) == int(np.argmax(logits))
    unseeded = {Sampler(SamplingParams(temperature=1.0)).seed for _ in range(4)}
    assert len(unseeded) == 4


def test_parameter_validation():
    for bad in (dict(temperature=-1), dict(top_p=0.0), dict(top_p=1.5), dict(top_k=-1),
                dict(repetition_penalty=0.0)):
        with pytest.raises(ValueError):
            Sampler(SamplingParams(**bad))

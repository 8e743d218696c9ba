"""Pins the CPU restatement of the device samplers (fusor-ml/core/src/sampling) against the answers the reference's
own tests hold, hand-worked cases and what the mathematics fixes."""
import math

import numpy as np
import pytest

STANDARD, MIROSTAT2 = 0, 1


def test_reference_stored_answers(oracle):
    # fusor-ml/core/src/sampling/tests.rs:226-272: flat candidates (ids 3,2,1,0 after the tie rule), mu 10, random 0.8
    flat = np.ones(4, np.float32)
    r = oracle.sample_token(flat, MIROSTAT2, 4, tau=5.0, eta=0.1, random=0.8, mu=10.0)
    assert list(r["ids"]) == [3, 2, 1, 0] and r["token"] == 0
    # :275-318: top_p 0.5 keeps two of the four flat candidates; random 0.8 picks the second, id 2
    r = oracle.sample_token(flat, STANDARD, 4, top_p=0.5, min_p=0.0, random=0.8)
    assert r["token"] == 2
    # :192-223: Mirostat over the processed order, top_k 4, random 0 -> the first candidate
    vals = np.array([9.0, 8.5, 7.0, 6.0, 2.5, 0.25, -1.0, -3.0], np.float32)
    r = oracle.sample_token(vals, MIROSTAT2, 4, tau=5.0, eta=0.1, random=0.0, mu=10.0)
    assert r["token"] == 0 and list(r["ids"]) == [0, 1, 2, 3]
    # models/kalosm-llama/src/sampler.rs:404-441: min_p 0.1 leaves only the top candidate of 0, -3, -4, -5
    logits = np.array([-5.0, -4.0, -3.0, 0.0], np.float32)
    for rnd in (0.0, 0.5, 0.999):
        assert oracle.sample_token(logits, STANDARD, 4, min_p=0.1, random=rnd)["token"] == 3
    # sampler.rs:384-401: top_p 0.5 restricts flat logits to ids 3 and 2 whatever the random number
    seen = {oracle.sample_token(flat, STANDARD, 4, top_p=0.5, random=rnd)["token"] for rnd in np.linspace(0, 0.999, 64)}
    assert seen == {2, 3}


def test_reference_mirostat_case_worked_by_hand(oracle):
    # tests.rs:321-368: values 9, 7.5, 7, 4, 3.5, 1; top_k 5; mu 3; random 0.65.  Weights 1, e^-1.5, e^-2, e^-5, e^-5.5;
    # probabilities 0.7303, 0.1630, 0.0988: the third has surprise 3.34 > 3, so two candidates stay; their weight is
    # 1.2231, the threshold 0.795 is reached by the first -> id 0.  mu' = 3 - 0.1 * (-log2(1 / 1.2231) - 5).
    vals = np.array([9.0, 7.5, 7.0, 4.0, 3.5, 1.0], np.float32)
    r = oracle.sample_token(vals, MIROSTAT2, 5, tau=5.0, eta=0.1, random=0.65, mu=3.0)
    assert r["token"] == 0
    assert r["mu"] == pytest.approx(3.0 - 0.1 * (math.log2(1.0 + math.exp(-1.5)) - 5.0), rel=1e-6)
    # random 0.9: threshold 1.1008 > 1 -> the second candidate, id 1
    r = oracle.sample_token(vals, MIROSTAT2, 5, tau=5.0, eta=0.1, random=0.9, mu=3.0)
    assert r["token"] == 1
    assert r["mu"] == pytest.approx(3.0 - 0.1 * (-math.log2(math.exp(-1.5) / (1.0 + math.exp(-1.5))) - 5.0), rel=1e-6)


def test_processors_case_of_the_reference_worked_by_hand(oracle):
    # tests.rs:61-136: temperature 0.5, penalty 2, previous {0, 3, 9}: ids 0, 3, 9 are halved (all positive), then
    # everything doubles: 4 -> 4, 8 -> 8, 7 -> 7; NaN and -inf drop out.
    values = np.array([4.0, -2.0, 3.5, 8.0, np.nan, 1.0, 5.0, -1.5, 6.5, 7.0, -np.inf, 0.5], np.float32)
    r = oracle.sample_token(values, STANDARD, 5, temperature=0.5, repetition_penalty=2.0, previous=[0, 3, 9], random=0.0)
    assert list(r["ids"]) == [8, 6, 3, 9, 2]
    assert list(r["values"]) == [13.0, 10.0, 8.0, 7.0, 7.0]
    # a negative repeated logit is multiplied: -2 * 2 / 0.5 = -8; a penalty of 1 or less does nothing
    r = oracle.sample_token(values, STANDARD, 10, temperature=0.5, repetition_penalty=2.0, previous=[1], random=0.0)
    assert dict(zip(r["ids"].tolist(), r["values"].tolist()))[1] == -8.0
    r = oracle.sample_token(values, STANDARD, 11, temperature=0.0, repetition_penalty=0.5, previous=[1, 3], random=0.0)
    got = dict(zip(r["ids"].tolist(), r["values"].tolist()))
    assert got[1] == -2.0 and got[3] == 8.0            # temperature 0 leaves the logits alone
    assert r["ids"][-1] == 0xFFFFFFFF                    # ten finite values only
    none = oracle.sample_token(np.array([np.nan, np.inf], np.float32), STANDARD, 4, random=0.3)
    assert none["token"] is None and none["status"] == 2


def test_sampled_frequencies_follow_the_softmax(oracle):
    rng = np.random.default_rng(5)
    logits = rng.normal(0, 1.5, 40).astype(np.float32)
    k = 8
    order = np.argsort(-logits.astype(np.float64), kind="stable")[:k]
    p = np.exp(logits[order].astype(np.float64) - logits[order[0]])
    p /= p.sum()
    draws = 4000
    counts = np.zeros(k)
    for u in (np.arange(draws) + 0.5) / draws:       # stratified uniforms: counts must match p to 1 / draws per slot
        t = oracle.sample_token(logits, STANDARD, k, random=float(u))["token"]
        counts[list(order).index(t)] += 1
    assert np.abs(counts / draws - p).max() < 2.0 / draws
    # the same through Mirostat with a mu no candidate exceeds
    counts = np.zeros(k)
    for u in (np.arange(draws) + 0.5) / draws:
        t = oracle.sample_token(logits, MIROSTAT2, k, random=float(u), mu=100.0)["token"]
        counts[list(order).index(t)] += 1
    assert np.abs(counts / draws - p).max() < 2.0 / draws


def test_top_p_and_min_p_cut_where_the_cumulative_weight_says(oracle):
    logits = np.log(np.array([0.5, 0.25, 0.125, 0.075, 0.05], np.float64)).astype(np.float32)
    for top_p, keep in ((0.4, 1), (0.6, 2), (0.8, 3), (0.9, 4), (1.0, 5)):
        seen = {oracle.sample_token(logits, STANDARD, 5, top_p=top_p, random=float(u))["token"]
                for u in np.linspace(0, 0.9999, 200)}
        assert seen == set(range(keep)), (top_p, seen)
    # min_p compares exp(value - max): 0.3 keeps weights 1 and 0.5 only; top_p then works on what is left
    seen = {oracle.sample_token(logits, STANDARD, 5, min_p=0.3, random=float(u))["token"] for u in np.linspace(0, 0.9999, 200)}
    assert seen == {0, 1}
    seen = {oracle.sample_token(logits, STANDARD, 5, min_p=0.3, top_p=0.5, random=float(u))["token"]
            for u in np.linspace(0, 0.9999, 200)}
    assert seen == {0}                                  # 0.5 of the filtered 1.5 is reached by the first weight


def test_mirostat_cutoff_and_update_closed_form(oracle):
    # two candidates with probabilities 0.8 / 0.2: surprises 0.32 and 2.32
    logits = np.log(np.array([0.8, 0.2])).astype(np.float32)
    r = oracle.sample_token(logits, MIROSTAT2, 2, tau=3.0, eta=0.25, random=0.95, mu=5.0)
    assert r["token"] == 1 and r["mu"] == pytest.approx(5.0 - 0.25 * (-math.log2(0.2) - 3.0), rel=1e-5)
    # mu 1 cuts the second candidate off (the cutoff never drops below one candidate); the survivor has probability 1
    r = oracle.sample_token(logits, MIROSTAT2, 2, tau=3.0, eta=0.25, random=0.95, mu=1.0)
    assert r["token"] == 0 and r["mu"] == pytest.approx(1.0 - 0.25 * (0.0 - 3.0), rel=1e-6)
    r = oracle.sample_token(logits, MIROSTAT2, 2, tau=3.0, eta=0.25, random=0.95, mu=0.1)
    assert r["token"] == 0

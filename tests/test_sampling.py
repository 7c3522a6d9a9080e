"""CPU tests that pin the numpy restatement of the sampler and its random numbers (oracle/sampling.py) against what is
known from outside it: published Threefry vectors, sha256, closed forms, brute force in float64, and statistics."""
import hashlib

import numpy as np
import pytest

import oracle as orc
from oracle import sampling as S

RNG = np.random.default_rng(31)


def test_threefry_known_answers():
    """The three known-answer vectors of Threefry-2x32-20 from the Random123 distribution (also used by JAX's tests)."""
    kat = [((0, 0), (0, 0), (0x6B200159, 0x99BA4EFE)),
           ((0xFFFFFFFF, 0xFFFFFFFF), (0xFFFFFFFF, 0xFFFFFFFF), (0x1CB996FC, 0xBB002BE7)),
           ((0x243F6A88, 0x85A308D3), (0x13198A2E, 0x03707344), (0xC4923A9C, 0x483DF7A0))]
    for ctr, key, want in kat:
        y0, y1 = S.threefry2x32(np.uint32(ctr[0]), np.uint32(ctr[1]), key[0], key[1])
        assert (int(y0), int(y1)) == want
    # vectorised over counters == one at a time
    c = np.arange(5, dtype=np.uint32)
    y0, y1 = S.threefry2x32(c, c + np.uint32(7), 123, 456)
    for i in range(5):
        a, b = S.threefry2x32(np.uint32(i), np.uint32(i + 7), 123, 456)
        assert (int(a), int(b)) == (int(y0[i]), int(y1[i]))


def test_device_key_is_the_tail_of_sha256_of_the_device_count():
    assert hashlib.sha256(bytes(4)).hexdigest() == "df3f619804a92fdb4057192dc43dd748ea778adc52bc498ce80524c014b81119"
    assert S.device_key0(0) == 0x14B81119                     # big-endian integer mod 2^32 = the last four bytes
    assert S.device_key0(1) == int(hashlib.sha256(b"\x00\x00\x00\x01").hexdigest()[-8:], 16)


def test_rand_is_23_mantissa_bits_of_the_low_word():
    for seed, counter in ((0, 0), (42, 0), (42, 1), (7, 2 ** 32 - 1)):
        y0, _ = S.threefry2x32(np.uint32(counter & 0xFFFFFFFF), np.uint32((counter + 1) & 0xFFFFFFFF), S.device_key0(0), seed)
        u = S.rand_f32(seed, counter)
        assert u == np.float32((int(y0) >> 9) * 2.0 ** -23) and 0.0 <= u < 1.0
    us = np.array([S.rand_f32(1234, c) for c in range(20000)])
    hist = np.histogram(us, bins=16, range=(0, 1))[0]
    assert ((hist - 1250.0) ** 2 / 1250.0).sum() < 45.0        # chi-square, 15 degrees of freedom: 45 is far in the tail
    assert len(set(us.tolist())) > 19900


def _cumsum_by_definition(x):
    """tensor.ts:2629-2641 with python loops"""
    x = [np.float32(v) for v in x]
    n = len(x)
    if n <= 512:
        out, acc = [], np.float32(0)
        for v in x:
            acc = np.float32(acc + v); out.append(acc)
        return np.array(out, np.float32)
    pad = (-n) % 256
    xp = [np.float32(0)] * pad + x
    within, totals = [], []
    for c in range(len(xp) // 256):
        acc = np.float32(0)
        for v in xp[c * 256:(c + 1) * 256]:
            acc = np.float32(acc + v); within.append(acc)
        totals.append(acc)
    base, acc = [], np.float32(0)
    for t in totals:
        base.append(acc); acc = np.float32(acc + t)
    return np.array([np.float32(within[i] + base[i // 256]) for i in range(len(xp))], np.float32)[pad:]


@pytest.mark.parametrize("n", [1, 5, 256, 512, 513, 700, 1024, 2049])
def test_cumsum_is_the_two_level_scheme(n):
    x = RNG.random(n).astype(np.float32)
    got = S.cumsum(x)
    assert np.array_equal(got, _cumsum_by_definition(x))
    assert np.allclose(got, np.cumsum(x.astype(np.float64)), rtol=1e-5)
    assert abs(float(S.seq_sum(x)) - float(x.astype(np.float64).sum())) <= 1e-5 * n


def _first_above(cdf64, u):
    return int(np.sum(u >= cdf64))


def test_multinomial_brute_force_and_frequencies():
    w = np.float32([0.1, 0.2, 0.3, 0.4])
    cdf = np.cumsum(w.astype(np.float64)) / w.astype(np.float64).sum()
    for u in np.linspace(0.003, 0.997, 199):                   # none of these is within 1e-3 of a boundary
        assert S.multinomial(w, np.float32(u)) == _first_above(cdf, u)
    assert S.multinomial(w, np.float32(0.0)) == 0 and S.multinomial(w, np.float32(0.0999)) == 0 and S.multinomial(w, np.float32(0.1001)) == 1
    draws = np.array([S.multinomial(w, S.rand_f32(5, c)) for c in range(20000)])
    freq = np.bincount(draws, minlength=4) / 20000.0
    assert np.all(np.abs(freq - w) < 0.012)
    # unnormalised weights and zeros: zero-weight entries are never drawn
    w2 = np.float32([0, 3, 0, 1, 0])
    assert set(S.multinomial(w2, np.float32(u)) for u in np.linspace(0.001, 0.999, 97)) == {1, 3}


def test_sample_full_vocabulary_path():
    n = 1000
    logits = (RNG.standard_normal(n) * 3).astype(np.float32)
    temp = 0.95
    p64 = np.exp((logits.astype(np.float64) / temp) - (logits.astype(np.float64) / temp).max())
    cdf = np.cumsum(p64) / p64.sum()
    checked = 0
    for c in range(300):
        u = S.rand_f32(9, c)
        if np.min(np.abs(cdf - float(u))) < 1e-5:
            continue                                            # too close to a boundary for float64 to be the judge
        assert S.sample(logits, temp, 0, 0.0, 0.0, 0.0, u) == _first_above(cdf, float(u))
        checked += 1
    assert checked > 250
    assert S.sample(logits, 0.0, 0, 0.0, 0.0, 0.0, np.float32(0.7)) == int(np.argmax(logits))     # temperature 0 -> argmax
    assert np.allclose(S.softmax_t(logits, temp), p64 / p64.sum(), rtol=2e-5, atol=1e-9)
    # NaN logits are never drawn
    bad = logits.copy(); bad[::3] = np.nan
    assert all(S.sample(bad, temp, 0, 0.0, 0.0, 0.0, S.rand_f32(1, c)) % 3 != 0 for c in range(200))


def test_sample_top_k_and_top_p():
    n = 600
    logits = (RNG.standard_normal(n) * 2).astype(np.float32)
    order = np.argsort(-logits, kind="stable")
    top5 = set(order[:5].tolist())
    toks = [S.sample(logits, 0.9, 5, 1.0, 0.0, 0.0, S.rand_f32(3, c)) for c in range(4000)]
    assert set(toks) == top5                                                       # p = 1 keeps all k
    pr = S.softmax_t(logits, 0.9).astype(np.float64)[order[:5]]
    freq = np.array([toks.count(int(t)) for t in order[:5]]) / 4000.0
    assert np.all(np.abs(freq - pr / pr.sum()) < 0.03)
    assert all(S.sample(logits, 0.9, 1, 1.0, 0.0, 0.0, S.rand_f32(3, c)) == int(order[0]) for c in range(50))    # k = 1
    # top p: an entry stays when the mass from it downwards reaches 1 - p, i.e. the smallest head whose mass reaches p
    crafted = np.log(np.float32([0.5, 0.3, 0.1, 0.05, 0.03, 0.02]))
    seen = set(S.sample(crafted, 1.0, 4, 0.6, 0.0, 0.0, S.rand_f32(4, c)) for c in range(500))
    assert seen == {0, 1}
    seen = set(S.sample(crafted, 1.0, 4, 0.85, 0.0, 0.0, S.rand_f32(4, c)) for c in range(800))
    assert seen == {0, 1, 2}
    # ties: the k largest by repeated argmax take the lowest indices first
    tied = np.zeros(10, np.float32)
    assert set(S.sample(tied, 1.0, 3, 1.0, 0.0, 0.0, S.rand_f32(5, c)) for c in range(300)) == {0, 1, 2}
    with pytest.raises(ValueError):
        S.sample(logits, 1.0, n + 1, 0.5, 0.0, 0.0, np.float32(0.5))
    with pytest.raises(ValueError):
        S.sample(logits, 1.0, 0, 1.5, 0.0, 0.0, np.float32(0.5))


def test_sample_alpha_penalties():
    n = 50
    logits = np.zeros(n, np.float32); logits[7] = 6.0
    cnt = np.zeros(n, np.int32)
    first = S.sample(logits, 1.0, 0, 0.0, 4.0, 0.5, np.float32(0.5), cnt)
    assert first == 7 and cnt[7] == 1 and cnt.sum() == 1
    # the penalty as llama.ts:147 writes it: count * af + (count >= 0) * ap, the second term for EVERY entry
    pen = cnt.astype(np.float32) * np.float32(4.0) + np.float32(0.5)
    want = S.softmax_t(logits - pen, 1.0)
    u = np.float32(0.5)
    assert S.sample(logits, 1.0, 0, 0.0, 4.0, 0.5, u, cnt.copy()) == S.multinomial(want, u)
    for _ in range(3):
        S.sample(logits, 1.0, 0, 0.0, 4.0, 0.5, np.float32(0.01), cnt)
    assert cnt.sum() == 4

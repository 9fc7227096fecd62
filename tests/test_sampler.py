"""Top-p sampling (src/main.rs:74-137) and the turn loop around it (:325-378).

The CPU checker's sampler is pinned by what the algorithm's definition fixes: with the draw r swept over a fine
grid the share of draws that land on a token is its renormalised nucleus probability (fp64 softmax), the nucleus
is the shortest prefix of the probability-sorted tokens whose mass reaches top_p, ties keep index order, the
penalty divides the recent tokens' logits whatever their sign.  The library's sampler must then return exactly
what the checker returns."""
import numpy as np
import pytest

from lumen_amd import ops
from oracle import lumen_oracle as lo

RNG = np.random.default_rng(11)


def nucleus_fp64(logits, temperature, top_p, penalty=1.0, recent=()):
    z = np.asarray(logits, np.float64).copy()
    if penalty > 1.0:
        for t in recent:
            z[t] /= penalty
    z /= max(temperature, 1e-5)
    p = np.exp(z - z.max())
    p /= p.sum()
    order = np.argsort(-p, kind="stable")
    cum = np.cumsum(p[order])
    cut = int(np.searchsorted(cum, min(max(top_p, 1e-6), 1.0) - 1e-12) + 1)
    cut = min(cut, len(p))
    keep = order[:cut]
    return keep, p[keep] / p[keep].sum()


@pytest.mark.parametrize("n,temperature,top_p", [(50, 1.0, 1.0), (200, 0.8, 0.9), (37, 1.7, 0.5), (1000, 0.3, 0.95)])
def test_checker_sampler_is_the_inverse_cdf_of_the_nucleus(n, temperature, top_p):
    logits = RNG.normal(0, 2.0, n).astype(np.float32)
    keep, q = nucleus_fp64(logits, temperature, top_p)
    grid = (np.arange(20000) + 0.5) / 20000
    picks = np.array([lo.sample_top_p(logits, temperature, top_p, 1.0, [], r) for r in grid])
    assert set(np.unique(picks)) <= set(keep.tolist())
    freq = np.array([(picks == t).mean() for t in keep])
    # a token whose nucleus mass straddles the top_p boundary can differ by what f32 rounding moves: compare on
    # the nucleus the fp64 definition gives, with the grid's resolution plus that slack
    assert np.abs(freq - q).max() < 3e-4 + 2e-3 * (len(keep) > 1) * q.min()
    # draws are monotone: a larger r never picks an earlier token of the sorted nucleus
    rank = {t: i for i, t in enumerate(keep.tolist())}
    r_sorted = [rank[t] for t in picks]
    assert all(a <= b for a, b in zip(r_sorted, r_sorted[1:]))


def test_checker_sampler_special_cases():
    logits = np.array([0.1, 2.0, -1.0, 2.0, 0.5], np.float32)
    # top_p -> 0: the most probable token; of two equal ones the lower index (stable sort)
    assert lo.sample_top_p(logits, 1.0, 0.0, 1.0, [], 0.99) == 1
    # r = 0 always picks the head of the nucleus, r = 1 its tail
    assert lo.sample_top_p(logits, 1.0, 1.0, 1.0, [], 0.0) == 1
    assert lo.sample_top_p(logits, 1.0, 1.0, 1.0, [], 1.0) == 2
    # tiny temperature = arg-max whatever r
    assert all(lo.sample_top_p(logits, 0.0, 1.0, 1.0, [], r) == (1 if r <= 0.5 else 3) for r in (0.0, 0.3, 0.7, 0.999))
    assert all(lo.sample_top_p(logits[:3], 0.0, 1.0, 1.0, [], r) == 1 for r in (0.0, 0.3, 0.999))
    # the penalty divides the logit: a positive one falls, a negative one rises (the reference's behaviour)
    x = np.array([3.0, 2.9, -0.2, -0.1], np.float32)
    assert lo.sample_top_p(x, 1.0, 0.0, 1.0, [], 0.5) == 0
    assert lo.sample_top_p(x, 1.0, 0.0, 1.5, [0], 0.5) == 1
    y = np.array([-3.0, -2.0, -4.0], np.float32)
    assert lo.sample_top_p(y, 1.0, 0.0, 1.0, [], 0.5) == 1
    assert lo.sample_top_p(y, 1.0, 0.0, 4.0, [0], 0.5) == 0
    # penalties <= 1 and out-of-range ids do nothing
    assert lo.sample_top_p(x, 1.0, 0.0, 1.0, [0], 0.5) == 0
    assert lo.sample_top_p(x, 1.0, 0.0, 2.0, [17], 0.5) == 0


@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 700, 32000])
def test_library_sampler_equals_the_checker(n):
    for trial in range(6):
        logits = RNG.normal(0, 1.0 + trial, n).astype(np.float32)
        if trial == 3:
            logits[: n // 2] = logits[0]  # many ties
        recent = RNG.integers(0, n, size=min(n, 20))
        for temperature, top_p, pen in [(0.8, 0.9, 1.05), (1.0, 1.0, 1.0), (0.05, 0.3, 2.0), (2.5, 0.999, 1.0), (1.0, 0.0, 1.0)]:
            for r in [0.0, 1e-7, 0.37, 0.5, 0.93, 0.9999999, 1.0]:
                want = lo.sample_top_p(logits, temperature, top_p, pen, recent, r)
                got = ops.sample_top_p(logits, temperature, top_p, pen, recent, r)
                assert got == want, (n, trial, temperature, top_p, pen, r)


def test_seeded_stream_is_uniform_and_repeatable():
    a, b = ops.rand01_stream(42, 20000), ops.rand01_stream(42, 20000)
    assert np.array_equal(a, b) and not np.array_equal(a, ops.rand01_stream(43, 20000))
    assert a.min() >= 0.0 and a.max() < 1.0
    hist = np.histogram(a, bins=20, range=(0, 1))[0] / a.size
    assert np.abs(hist - 0.05).max() < 0.006 and abs(a.mean() - 0.5) < 0.01
    # splitmix64 known answers: first outputs for state 0 are 0xe220a8397b1dcdaf, 0x6e789e6aa1b965f4
    assert np.array_equal(ops.rand01_stream(0, 2), np.array([(0xe220a8397b1dcdaf >> 40) / 2 ** 24, (0x6e789e6aa1b965f4 >> 40) / 2 ** 24], np.float32))


@pytest.mark.gpu
def test_generate_turn_follows_the_reference_loop():
    from lumen_amd import synth
    from lumen_amd.models import LlamaModel

    cfg = dict(vocab_size=500, hidden_size=128, intermediate_size=352, num_hidden_layers=2, num_attention_heads=4,
               num_key_value_heads=2, rms_norm_eps=1e-5, max_seq_len=96, rope_theta=10000.0)
    params = synth.make_params(cfg, seed=9, std=0.2, gains_one=False)
    gpu = LlamaModel(cfg)
    gpu.load_params(params)
    ora = lo.Llama(cfg, params)
    turn1 = synth.make_tokens(11, cfg["vocab_size"], seed=9)
    kw = dict(temperature=0.8, top_p=0.9, repetition_penalty=1.05, recent_window=16)

    def checker_turn(new, history, max_gen, seed, stop_ids):
        """main.rs:325-378 on the CPU checker with the same draws; also returns how close each draw came to a
        boundary of the inverse CDF (a GPU logit difference of 1e-4 can only flip a pick that close)."""
        draws = ops.rand01_stream(seed, max_gen)
        hist = list(history) + list(new)
        _, lg = ora.forward(np.asarray(new))
        lg = lg[-1]
        out = []
        for g in range(max_gen):
            recent = hist[-kw["recent_window"]:]
            nxt = lo.sample_top_p(lg, kw["temperature"], kw["top_p"], kw["repetition_penalty"], recent, draws[g])
            if nxt in stop_ids:
                break
            hist.append(nxt)
            out.append(nxt)
            _, lg = ora.forward(np.array([nxt]))
            lg = lg[0]
            if ora.kv_len + 2 >= cfg["max_seq_len"]:
                break
        return out

    got1 = gpu.generate_turn(turn1, max_gen=12, seed=5, **kw)
    want1 = checker_turn(turn1, [], 12, 5, [])
    assert got1.tolist() == want1 and gpu.kv_len == ora.kv_len == 11 + 12
    # second turn into the live cache, history reaching into the first; a stop id ends it early
    hist = turn1.tolist() + want1
    turn2 = synth.make_tokens(7, cfg["vocab_size"], seed=10)
    free = checker_turn(turn2, hist, 10, 6, [])
    ora.reset()
    ora.forward(np.asarray(hist))  # rebuild the checker's cache up to the end of turn 1
    stop = [free[4]]
    want2 = checker_turn(turn2, hist, 10, 6, stop)
    assert want2 == free[:free.index(stop[0])]
    got2 = gpu.generate_turn(turn2, history=hist, max_gen=10, seed=6, stop_ids=stop, **kw)
    assert got2.tolist() == want2
    # a turn that would run into the end of the cache is refused before anything is fed (main.rs:266)
    from lumen_amd import _lib
    with pytest.raises(_lib.LumenError) as e:
        gpu.generate_turn(synth.make_tokens(70, cfg["vocab_size"], seed=3), max_gen=4, **kw)
    assert e.value.status == _lib.ERR_KV_OVERFLOW
    # generation stops two short of the cache's end (main.rs:370-372)
    gpu.reset_kv_caches()
    out = gpu.generate_turn(synth.make_tokens(60, cfg["vocab_size"], seed=4), max_gen=200, seed=1, **kw)
    assert gpu.kv_len == cfg["max_seq_len"] - 2 and len(out) == cfg["max_seq_len"] - 2 - 60

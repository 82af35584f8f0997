"""Pins for the CPU oracle (no GPU).  The reference ships no tests, golden vectors or
fixtures for this path, so each part of the oracle is pinned by what the mathematics
fixes: closed forms, known-answer vectors of the published generator, float64 / exact
integer brute force, special cases that reduce to library routines, and the literal fp32
emulation of the reference kernel's thread layout.  A plausible mistake (dropped term,
wrong sign or index, off-by-one in a shift) fails at least one of these."""
import math
from fractions import Fraction

import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from tests import helpers as H

F32 = np.float32


def bits(x):
    return np.asarray(x, dtype=np.float32).view(np.uint32)


# ------------------------------------------------------------------ sf / scale
def test_sf_closed_form(oracle):
    L = oracle.lib()
    fmax = float(np.finfo(np.float32).max)
    assert L.rs_oracle_sf(float("nan")) == 0.0
    assert L.rs_oracle_sf(float("inf")) == fmax
    assert L.rs_oracle_sf(float("-inf")) == -fmax
    for v in (0.0, -0.0, 1.5, -3.25e30, 1e-45):
        assert L.rs_oracle_sf(v) == float(F32(v))


def test_scale_order_of_operations(oracle):
    """x = sf((sf(l) - pen) * c): the penalty is subtracted BEFORE the temperature scale
    (sampling.cu:220), in fp32, one rounding per operation."""
    L = oracle.lib()
    rng = np.random.default_rng(0)
    for _ in range(2000):
        l, p, c = F32(rng.normal() * 10), F32(rng.exponential()), F32(rng.uniform(0.1, 5))
        exp = F32(F32(l - p) * c)
        assert L.rs_oracle_scale(float(l), float(p), 1, float(c)) == float(exp)
        assert L.rs_oracle_scale(float(l), 123.0, 0, float(c)) == float(F32(l * c))
    fmax = float(np.finfo(np.float32).max)
    assert L.rs_oracle_scale(1.0, float("-inf"), 1, 2.0) == fmax          # masked with -inf penalty
    assert L.rs_oracle_scale(1.0, float("inf"), 1, 2.0) == -fmax
    assert L.rs_oracle_scale(float("inf"), float("inf"), 1, 2.0) == -fmax  # sf(inf)=FLT_MAX, minus inf
    assert L.rs_oracle_scale(float("nan"), 0.0, 1, 2.0) == 0.0


# ------------------------------------------------------------------ e = 2^(x - M)
def test_e_bits_accuracy_monotone_and_anchors(oracle):
    rng = np.random.default_rng(1)
    for M in (0.0, 3.0, -7.0, 1000.0):
        x = np.sort((M + 1 - np.abs(rng.normal(size=6000) * 9)).astype(np.float32))
        x = x[x < M + 1]                                    # floor(max) = M means every x < M + 1
        b = oracle.e_bits(x, M)
        e = b.view(np.float32).astype(np.float64)
        ref = np.exp2(x.astype(np.float64) - M)
        live = ref >= 2.0 ** -40
        rel = np.abs(e[live] - ref[live]) / ref[live]
        assert rel.max() < 2.0 * 2.0 ** -23, rel.max()     # within 2 ulp, as the reference's exp2f
        assert np.all(b[~live] == 0)                       # flushed to zero below 2^-40: dead tokens
        assert np.all(np.diff(b.astype(np.int64)) >= 0)    # monotone in x
        assert b.max() < 0x40000000                        # e < 2
        assert b[live].min() >= 0x2B800000                 # nothing between 0 and 2^-40
    assert oracle.e_bits(F32([5.0]), 5.0)[0] == bits(F32(1.0))[()]
    for k in range(0, 41):
        assert oracle.e_bits(F32([-k]), 0.0)[0] == bits(F32(2.0 ** -k))[()]     # exact powers of two
    assert oracle.e_bits(F32([-40.5, -1e30, -3.4e38]), 0.0).tolist() == [0] * 3
    just_below = np.nextafter(F32(-40.0), F32(-np.inf))
    assert oracle.e_bits(np.array([just_below, -40.0], dtype=np.float32), 0.0).tolist() == [0, 0x2B800000]


def test_e_significand_does_not_depend_on_the_maximum(oracle):
    """Shifting M by an integer only moves the exponent field: a slice can be worked with its own
    maximum and re-based later."""
    x = (np.random.default_rng(2).normal(size=4000) * 6).astype(np.float32)
    x = x[x < 20]
    b0 = oracle.e_bits(x, 20.0)
    for d in (1, 2, 7, 19):
        b1 = oracle.e_bits(x, 20.0 + d)
        rebased = b0.astype(np.int64) - (d << 23)
        rebased[rebased < 0x2B800000] = 0                  # what falls below 2^-40 of the new frame is dead
        assert np.array_equal(b1.astype(np.int64), rebased)


def test_e_monotone_across_every_octave_boundary(oracle):
    """poly(f -> 1) stays below 2 * poly(0): the floats on both sides of each integer are ordered."""
    for k in range(-39, 1):
        lo = np.nextafter(F32(k), F32(-np.inf))
        hi = np.nextafter(F32(k), F32(np.inf))
        b = oracle.e_bits(np.array([lo, F32(k), hi], dtype=np.float32), 0.0)
        assert b[0] <= b[1] <= b[2]
    tiny = oracle.e_bits(F32([-1e-10]), -1.0)[0]           # f rounds to 1.0: poly(1) < 2
    assert tiny < 0x40000000 and tiny >= bits(F32(1.999))[()]


# ------------------------------------------------------------------ exact weights
def test_w_is_e_times_2_pow_63(oracle):
    rng = np.random.default_rng(2)
    b = np.concatenate([oracle.e_bits((-np.abs(rng.normal(size=3000) * 15)).astype(np.float32), 0.0),
                        bits(F32([1.0, 1.5, 1.9999999, 2.0 ** -40, 2.0 ** -17, 0.75]))])
    w = oracle.w_of(b)
    for bi, wi in zip(b, w):
        exact = Fraction(float(np.uint32(bi).view(np.float32))) * 2 ** 63
        assert exact.denominator == 1 and int(wi) == exact.numerator == oracle.lib().rs_oracle_w(int(bi))
    assert int(w[b > 0].min()) == 2 ** 23 and int(w.max()) < 2 ** 64
    assert (b == 0).any() and np.all(w[b == 0] == 0)       # dead tokens weigh nothing


@settings(max_examples=300, deadline=None)
@given(st.floats(min_value=0.0, max_value=1.0, width=32), st.integers(min_value=1, max_value=2 ** 84))
def test_ceil_mul_exact(f, s):
    from oracle import oracle as O
    got = O.ceil_mul(f, s)
    if f <= 0.0:
        assert got == 1
    else:
        exact = math.ceil(Fraction(f) * s)
        assert got == min(max(exact, 1), s)


@settings(max_examples=200, deadline=None)
@given(st.integers(min_value=0, max_value=2 ** 64 - 1), st.integers(min_value=1, max_value=2 ** 84))
def test_r_from_bits_exact(u, s):
    from oracle import oracle as O
    assert O.r_from_bits(u, s) == (u * s) // 2 ** 64 + 1


# ------------------------------------------------------------------ Philox
def test_philox_known_answers(oracle):
    """Random123 known-answer vectors for philox4x32-10."""
    assert oracle.philox([0] * 4, [0] * 2) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert oracle.philox([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert oracle.philox([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0]) == \
        [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]


def test_philox_stream_layout(oracle):
    """curand_init(seed, row, 0) layout (sampling.cu:137): key = seed, counter = (draw, 0, row, 0).
    First words for seed 0: row 0 6627e8d5, row 1 844515e1, row 2 0661d677; second draw of row 0 f8e4cca4."""
    assert oracle.philox_draw(0, 0, 0)[:2] == [0x6627E8D5, 0xE169C58D]
    assert oracle.philox_draw(0, 1, 0)[:2] == [0x844515E1, 0xF08D6EAA]
    assert oracle.philox_draw(0, 2, 0)[:2] == [0x0661D677, 0xB6826759]
    assert oracle.philox_draw(0, 0, 1)[:2] == [0xF8E4CCA4, 0x5CB200DB]
    st_ = oracle.rng_init(0x1122334455667788, 3)
    assert st_[2, 0] == 0x55667788 and st_[2, 1] == 0x11223344 and st_[2, 4] == 2 and st_[2, 2] == 0


# ------------------------------------------------------------------ host normalisation
@pytest.mark.parametrize("temp,k,p,V,exp", [
    (1.0, -1, 0.5, 131072, (131072, 0.5)), (1.0, 0, 0.5, 1024, (1024, 0.5)), (1.0, 2000, 0.5, 1024, (1024, 0.5)),
    (1.0, 50, 1.5, 1024, (50, 1.0)), (1.0, 50, -0.1, 1024, (50, 1.0)), (1.0, 50, 0.0, 1024, (1, 1.0)),
    (0.8, 50, 0.9, 152064, (50, float(F32(0.9)))),
])
def test_normalisation_table(oracle, temp, k, p, V, exp):
    """sampling.cu:480-486 / :1005-1011."""
    c, kk, pp = oracle.normalize(temp, k, p, V)
    assert (kk, pp) == exp
    assert c == float(F32(math.log2(math.e) / temp))


@pytest.mark.parametrize("temp,V,B,T,what", [
    (1.0, 0, 1, 1, "vocabulary"), (1.0, 6, 1, 1, "vocabulary"), (1.0, 1048580, 1, 1, "vocabulary"),
    (1.0, 8, 0, 1, "B/T"), (1.0, 8, 1, 0, "B/T"), (0.0009, 8, 1, 1, "temperature"), (1001.0, 8, 1, 1, "temperature"),
    (float("nan"), 8, 1, 1, "temperature"),
])
def test_normalisation_errors(oracle, temp, V, B, T, what):
    with pytest.raises(ValueError, match=what):
        oracle.normalize(temp, -1, 0.5, V, B, T)


# ------------------------------------------------------------------ whole-row brute force
def brute_force_row(logits, c, top_k, top_p, u=None, u64=None, pen=None):
    """Independent restatement with Python integers and a sort (no search loop)."""
    from oracle import oracle as O
    L = O.lib()
    V = len(logits)
    x = [L.rs_oracle_scale(float(logits[i]), float(pen[i]) if pen is not None else 0.0, pen is not None, c)
         for i in range(V)]
    xmax = max(x)
    eb = O.e_bits(np.array(x, dtype=np.float32), math.floor(xmax))
    w = [Fraction(float(np.uint32(b).view(np.float32))) * 2 ** 63 for b in eb]
    assert all(v.denominator == 1 for v in w)
    w = [v.numerator for v in w]
    D = sum(w)
    P = min(max(math.ceil(Fraction(float(F32(top_p))) * D), 1), D)
    order = sorted(set(int(b) for b in eb if b > 0), reverse=True)     # dead tokens take no part
    cnt = mass = 0
    thr = order[-1]
    for val in order:
        members = [i for i in range(V) if eb[i] == val]
        cnt += len(members)
        mass += sum(w[i] for i in members)
        if cnt >= top_k or mass >= P:
            thr = val
            break
    n_gt = sum(1 for b in eb if b > thr)
    n_eq = sum(1 for b in eb if b == thr)
    G = sum(w[i] for i in range(V) if eb[i] > thr)
    w_thr = (Fraction(float(np.uint32(thr).view(np.float32))) * 2 ** 63).numerator
    w_tie = min(w_thr, (P - G) // n_eq if P > G else 0, (w_thr * (top_k - n_gt)) // n_eq if top_k > n_gt else 0)
    if w_tie == 0 and G == 0:
        w_tie = 1
    S = G + n_eq * w_tie
    if u is not None:
        r = min(max(math.ceil(Fraction(float(F32(u))) * S), 1), S) if u > 0 else 1
    else:
        r = (u64 * S) // 2 ** 64 + 1
    cdf, idx = 0, -1
    for i in range(V):
        cdf += w[i] if eb[i] > thr else (w_tie if eb[i] == thr else 0)
        if cdf >= r:
            idx = i
            break
    return dict(xmax=xmax, D=D, P=P, thr_bits=thr, n_gt=n_gt, n_eq=n_eq, G=G, w_tie=w_tie, S=S, r=r, index=idx)


CASES = [
    (64, 1.0, -1, 0.5), (64, 1.0, 5, 1.0), (256, 0.7, 10, 0.9), (256, 1.0, 256, 1.0), (256, 1.0, 1, 1.0),
    (128, 2.0, -1, 0.0), (512, 1.0, 50, 0.3), (128, 1.0, -1, 1e-30), (128, 1.0, 127, 1.0),
]


@pytest.mark.parametrize("V,temp,k,p", CASES)
def test_row_against_integer_brute_force(oracle, V, temp, k, p):
    rng = np.random.default_rng(V + int(temp * 10) + max(k, 0))
    for trial in range(6):
        kind = trial % 3
        lg = (rng.standard_normal(V) * 3).astype(np.float32) if kind == 0 else \
             rng.integers(0, 4, V).astype(np.float32) if kind == 1 else rng.random(V, dtype=np.float32)
        c, kk, pp = oracle.normalize(temp, k, p, V)
        u = float(F32(1.0 - rng.random()))
        got = oracle.sample_row(lg, c, kk, pp, u=u)
        exp = brute_force_row(lg, c, kk, pp, u=u)
        for key, val in exp.items():
            assert got[key] == val, (key, got[key], val, trial)
        u64 = int(rng.integers(0, 2 ** 63)) * 2 + 1
        got = oracle.sample_row(lg, c, kk, pp, u64=u64)
        assert got["index"] == brute_force_row(lg, c, kk, pp, u64=u64)["index"]


def test_search_loop_equals_definition_on_baseline_shapes(oracle):
    """The literal quaternary search (sampling.cu:261-329) lands on the definitional threshold
    'largest t with count >= top_k or mass >= P' (sort-based) on the BASELINE configurations."""
    cfgs = [(H.logits_uniform(1, 131072, 0), 1.0, -1, 0.5), (H.logits_normal(1, 262144, 3.0, 3), 1.0, -1, 0.3),
            (H.logits_spiked(2, 152064, seed=4), 0.8, 50, 0.9), (H.logits_normal(1, 1048576, 1.5, 7), 1.0, 1024, 0.95)]
    for lg, temp, k, p in cfgs:
        V = lg.shape[1]
        c, kk, pp = oracle.normalize(temp, k, p, V)
        for row in lg:
            d = oracle.sample_row(row, c, kk, pp, u=0.5, want_e=True)
            assert oracle.thr_by_sort(d["e_bits"], kk, d["P"]) == d["thr_bits"]
            assert d["left_bits"] <= d["thr_bits"] and 4 <= d["rounds"] <= 24


# ------------------------------------------------------------------ special cases -> library routines
def test_greedy_and_top1_are_argmax(oracle):
    rng = np.random.default_rng(5)
    for _ in range(20):
        lg = rng.standard_normal(4096).astype(np.float32)
        for (k, p) in [(-1, 0.0), (1, 1.0)]:
            c, kk, pp = oracle.normalize(1.0, k, p, 4096)
            d = oracle.sample_row(lg, c, kk, pp, u=float(F32(rng.random() * 0.999 + 0.001)))
            assert d["index"] == int(np.argmax(lg)) and d["n_gt"] == 0 and d["n_eq"] == 1


def test_keep_everything(oracle):
    lg = H.logits_normal(1, 8192, 2.0, 9)[0]
    c, kk, pp = oracle.normalize(1.0, -1, 1.0, 8192)
    d = oracle.sample_row(lg, c, kk, pp, u=1.0, want_e=True)
    assert d["e_bits"].min() > 0                            # every token of this row is live
    assert d["thr_bits"] == d["e_bits"].min() and d["n_gt"] + d["n_eq"] == 8192 and d["rounds"] == 0
    assert d["S"] <= d["D"] and d["index"] == int(np.nonzero(d["e_bits"] >= d["thr_bits"])[0][-1])


def test_masked_tokens_are_never_returned(oracle):
    """A logit at -inf (cleaned to -FLT_MAX, sampling.cu:131-134) has exp2f(x - max) = 0 in the
    reference (sampling.cu:235,248): threshold * comp cannot give it weight, so it never comes back,
    whatever top_k and top_p are.  Here e is flushed to zero below 2^-40 of the maximum."""
    V = 1 << 16
    rng = np.random.default_rng(21)
    live_ids = np.sort(rng.choice(V, size=4, replace=False))
    for low in (-np.inf, -200.0, -41.0 / 1.4426950408889634 - 1.0):
        lg = np.full(V, low, dtype=np.float32)
        lg[live_ids] = rng.standard_normal(4).astype(np.float32)
        for k, p in [(-1, 1.0), (1000, 1.0), (-1, 0.999999), (5, 1.0)]:
            c, kk, pp = oracle.normalize(1.0, k, p, V)
            for u in (1.0, float(np.nextafter(F32(1.0), F32(0.0))), 0.9999999, 0.5, 1e-30):
                d = oracle.sample_row(lg, c, kk, pp, u=u, want_e=True)
                assert d["index"] in live_ids, (low, k, p, u, d["index"])
                assert d["thr_bits"] >= 0x2B800000 and d["n_gt"] + d["n_eq"] <= 4
                assert np.count_nonzero(d["e_bits"]) == 4 and d["S"] <= d["D"]
            # 64 random bits at their largest reach the last live token, not the tail of the row
            d = oracle.sample_row(lg, c, kk, pp, u64=2 ** 64 - 1)
            assert d["index"] in live_ids
            if k == -1 and p == 1.0:
                assert d["index"] == live_ids[-1]
    # fewer live tokens than top_k: the kept set is every live token
    lg = np.full(V, -np.inf, dtype=np.float32)
    lg[live_ids] = [0.0, 1.0, 2.0, 3.0]
    c, kk, pp = oracle.normalize(1.0, 50, 1.0, V)
    d = oracle.sample_row(lg, c, kk, pp, u=1.0)
    assert d["n_gt"] + d["n_eq"] == 4 and d["S"] == d["D"] and d["index"] == live_ids[-1]


def test_all_equal_logits_are_uniform_over_all_tokens(oracle):
    """Degenerate row (reference bench logit type 0): every token ties at the threshold and the pick is
    uniform over all V tokens, whatever top_k says (sampling.cu:261,365-371)."""
    V = 1024
    lg = np.zeros(V, dtype=np.float32)
    c, kk, pp = oracle.normalize(1.0, 10, 0.5, V)
    seen = set()
    for j in range(1, 65):
        d = oracle.sample_row(lg, c, kk, pp, u=j / 64.0)
        assert d["n_eq"] == V and d["n_gt"] == 0 and d["G"] == 0
        assert d["index"] == -(-d["r"] // d["w_tie"]) - 1          # ceil(r / w_tie) - 1: equal weights
        seen.add(d["index"])
    assert len(seen) == 64 and max(seen) == V - 1


def test_invariants_on_random_rows(oracle):
    rng = np.random.default_rng(11)
    for _ in range(40):
        V = int(rng.choice([64, 1000, 4096]))
        V -= V % 4
        lg = (rng.standard_normal(V) * rng.uniform(0.2, 6)).astype(np.float32)
        k = int(rng.integers(1, V + 1))
        p = float(rng.uniform(0.01, 1.0))
        c, kk, pp = oracle.normalize(float(rng.uniform(0.3, 3)), k, p, V)
        d = oracle.sample_row(lg, c, kk, pp, u=float(F32(1.0 - rng.random())), want_e=True)
        e, thr = d["e_bits"], d["thr_bits"]
        q = oracle.w_of(e).astype(object)
        assert d["n_gt"] < kk and sum(q[e > thr]) < d["P"]                 # the set above thr is insufficient
        assert d["n_gt"] + d["n_eq"] >= kk or sum(q[e >= thr]) >= d["P"]    # the set at thr is sufficient
        assert 0 <= d["w_tie"] <= int(oracle.w_of(np.array([thr], dtype=np.uint32))[0])
        assert d["S"] <= max(d["P"], d["G"] + d["n_eq"]) and 1 <= d["r"] <= d["S"]
        assert d["n_gt"] * 1 + 0 <= kk and e[d["index"]] >= thr           # never a dropped token
        if d["n_eq"] * d["w_tie"] > 0:
            assert d["n_gt"] + d["n_eq"] * d["w_tie"] / int(oracle.w_of(np.array([thr], dtype=np.uint32))[0]) <= kk + 1e-9


# ------------------------------------------------------------------ penalties
def test_penalty_update_closed_form(oracle):
    """pen <- fma(pen, decay, onehot * (pen == 0 ? presence : repetition)), switch on the pre-decay value."""
    V = 2048
    rng = np.random.default_rng(13)
    lg = (rng.standard_normal(V) * 2).astype(np.float32)
    pen = H.penalties_sparse(1, V, frac=0.3, seed=14)[0]
    for trial in range(8):
        before = pen.copy()
        c, kk, pp = oracle.normalize(0.8, 50, 0.9, V)
        d = oracle.sample_row(lg, c, kk, pp, u=float(F32(1.0 - rng.random())), penalties=pen,
                              presence=0.3, repetition=0.1, decay=0.95)
        i = d["index"]
        exp = (before.astype(np.float64) * np.float64(F32(0.95)))
        exp[i] += np.float64(F32(0.3)) if before[i] == 0 else np.float64(F32(0.1))
        assert np.array_equal(pen, exp.astype(np.float32))     # fma: one rounding of the exact value
        changed = np.nonzero(pen != (before * F32(0.95)))[0]
        assert list(changed) == [i]


def test_btv_reads_only_last_position(oracle):
    """(B,T,V) logits: only logits[:, T-1, :] is sampled (sampling.cu:176,202)."""
    B, T, V = 3, 4, 1024
    x = H.logits_normal(B * T, V, 2.0, 15).reshape(B, T, V)
    u = H.uniforms(B, 16)
    c, kk, pp = oracle.normalize(1.0, 20, 0.9, V, B, T)
    out3, _ = oracle.sample_batch(x, c, kk, pp, injected_u=u)
    out2, _ = oracle.sample_batch(np.ascontiguousarray(x[:, T - 1, :]), c, kk, pp, injected_u=u)
    assert np.array_equal(out3, out2)


# ------------------------------------------------------------------ distribution
def test_oracle_pick_chi_square(oracle):
    from scipy import stats
    V = 64
    lg = H.logits_normal(1, V, 1.5, 17)[0]
    c, kk, pp = oracle.normalize(1.0, 12, 0.95, V)
    d = oracle.sample_row(lg, c, kk, pp, u=0.5, want_e=True)
    e, thr = d["e_bits"], d["thr_bits"]
    w = np.where(e > thr, oracle.w_of(e).astype(np.float64), 0.0)
    w[e == thr] = float(d["w_tie"])
    n = 100000
    logits2d = np.repeat(lg[None, :], n, axis=0)
    rng = oracle.rng_init(99, n)
    out, _ = oracle.sample_batch(logits2d, c, kk, pp, rng=rng)
    counts = np.bincount(out, minlength=V)
    assert counts[w == 0].sum() == 0
    chi2, pval = stats.chisquare(counts[w > 0], n * w[w > 0] / w.sum())
    assert pval > 0.01
    assert np.all(rng[:, 2] == 1)       # every row's draw counter advanced by one

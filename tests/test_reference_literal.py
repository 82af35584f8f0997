"""The canonical oracle against a LITERAL fp32 emulation of the reference kernel (oracle/ref_literal.c:
1024 virtual threads, the reference's own reduction trees, its float masses and two-uniform strided
pick).  The two differ only where float rounding decides: exp2 is a polynomial in one and libm's in the
other, masses are integers in one and rounded float sums in the other.  So the kept sets must agree up
to the handful of tokens whose probability lies within rounding of the threshold, and the picks must
follow the same distribution.  Also here: the reference's claim about scan order (README.md:169-179,
monotonicity.py) on its own 32-lane block scan and on a 64-lane ladder."""
import numpy as np
import pytest

from tests import helpers as H

F32 = np.float32


def _kept_sets(oracle, lg, temp, k, p, variant):
    V = lg.shape[0]
    c, kk, pp = oracle.normalize(temp, k, p, V)
    can = oracle.sample_row(lg, c, kk, pp, u=0.5, want_e=True)
    lit = oracle.literal_row(lg, c, kk, pp, 0.5, 0.5, variant=variant, want_probs=True)
    kept_c = can["e_bits"] >= can["thr_bits"]
    kept_l = lit["probs"] >= F32(lit["threshold"])
    return can, lit, kept_c, kept_l


@pytest.mark.parametrize("name,lg,temp,k,p,variant", [
    ("C1", H.logits_uniform(1, 131072, 0)[0], 1.0, -1, 0.5, 1),
    ("C2", H.logits_normal(1, 262144, 3.0, 3)[0], 1.0, -1, 0.3, 1),
    ("C3", H.logits_spiked(1, 152064, seed=4)[0], 0.8, 50, 0.9, 0),
    ("C5", H.logits_normal(1, 1048576, 1.5, 7)[0], 1.0, 1024, 0.95, 0),
    ("small-topk", H.logits_normal(1, 4096, 2.0, 8)[0], 0.7, 10, 1.0, 0),
])
def test_kept_set_matches_literal_reference(oracle, name, lg, temp, k, p, variant):
    can, lit, kept_c, kept_l = _kept_sets(oracle, lg, temp, k, p, variant)
    diff = int(np.count_nonzero(kept_c != kept_l))
    n = int(kept_c.sum())
    # top-k bound rows must agree exactly; top-p bound rows up to float rounding of the mass
    if k > 0 and can["n_gt"] + can["n_eq"] <= k and can["n_eq"] == 1 and can["n_gt"] + 1 == k:
        assert diff == 0, (name, diff)
    assert diff <= max(2, n // 2000), (name, diff, n)
    # probabilities agree to a few ulp: e / D  vs  exp2f(x - max) / denom
    pc = can["e_bits"].view(np.float32).astype(np.float64) * 2.0 ** 63 / float(can["D"])
    live = lit["probs"] > 1e-30
    rel = np.abs(pc[live] - lit["probs"][live].astype(np.float64)) / lit["probs"][live]
    assert rel.max() < 2e-5, (name, rel.max())


def test_literal_tie_compensation_matches_integer_form(oracle):
    """comp = min(1, (top_p - sgtp)/(thr*neqk), (top_k - sgtk)/neqk)  (sampling.cu:368-371) against
    w_tie / q_thr of the canonical oracle, on rows with a tie group at the threshold."""
    V = 4096
    rng = np.random.default_rng(3)
    lg = rng.integers(0, 6, V).astype(np.float32)       # heavy ties
    for (k, p) in [(100, 1.0), (-1, 0.6), (700, 0.9)]:
        c, kk, pp = oracle.normalize(1.0, k, p, V)
        can = oracle.sample_row(lg, c, kk, pp, u=0.5)
        lit = oracle.literal_row(lg, c, kk, pp, 0.5, 0.5, variant=0)
        assert can["n_eq"] == lit["n_eq"] and can["n_gt"] == lit["n_gt"]
        q_thr = int(oracle.w_of(np.array([can["thr_bits"]], dtype=np.uint32))[0])
        assert abs(can["w_tie"] / q_thr - lit["comp"]) < 1e-4


def test_literal_and_canonical_picks_share_a_distribution(oracle):
    from scipy import stats
    V = 256
    lg = H.logits_normal(1, V, 1.5, 21)[0]
    c, kk, pp = oracle.normalize(1.0, 20, 0.9, V)
    can = oracle.sample_row(lg, c, kk, pp, u=0.5, want_e=True)
    e, thr = can["e_bits"], can["thr_bits"]
    w = np.where(e > thr, oracle.w_of(e).astype(np.float64), 0.0)
    w[e == thr] = float(can["w_tie"])
    rng = np.random.default_rng(22)
    n = 20000
    counts = np.zeros(V, dtype=np.int64)
    for _ in range(n):
        u1, u2 = F32(1.0 - rng.random()), F32(1.0 - rng.random())
        counts[oracle.literal_row(lg, c, kk, pp, float(u1), float(u2), variant=0)["index"]] += 1
    assert counts[w == 0].sum() == 0
    chi2, pval = stats.chisquare(counts[w > 0], n * w[w > 0] / w.sum())
    assert pval > 0.001


# ------------------------------------------------------------------ scan order
def _stress_rows(n_rows, width, seed):
    """monotonicity.py:3-4: random non-negative floats drawn as bit patterns below 0x70000000."""
    rng = np.random.default_rng(seed)
    return rng.integers(0, 0x70000000, size=(n_rows, width), dtype=np.int64).astype(np.uint32).view(np.float32)


def test_reference_block_scan_is_monotone_only_with_descending_ladder(oracle):
    rows = _stress_rows(300, 1024, 1)
    bad_desc = bad_asc = 0
    for r in rows:
        d, tot = oracle.literal_block_scan(r, descending=True)
        a, _ = oracle.literal_block_scan(r, descending=False)
        bad_desc += int(np.any(np.diff(d) < 0))
        bad_asc += int(np.any(np.diff(a) < 0))
        assert d[-1] == F32(tot)                                   # last element is the total, bit for bit
        ref = np.cumsum(r.astype(np.float64))
        assert np.all(np.abs(d.astype(np.float64) - ref) <= 1024 * 2.0 ** -23 * ref)
    assert bad_desc == 0            # 16,8,4,2,1 + serial combine: monotone (README.md:169)
    assert bad_asc > 0              # 1,2,4,8,16: the negative control must fail


def test_wave64_ladder_scan_order(oracle):
    rows = _stress_rows(4000, 64, 2)
    bad_desc = bad_asc = 0
    for r in rows:
        d = oracle.literal_wave64_scan(r, descending=True)      # 32,16,8,4,2,1
        a = oracle.literal_wave64_scan(r, descending=False)     # 1,2,...,32
        bad_desc += int(np.any(np.diff(d) < 0))
        bad_asc += int(np.any(np.diff(a) < 0))
        ref = np.cumsum(r.astype(np.float64))
        assert np.all(np.abs(d.astype(np.float64) - ref) <= 64 * 2.0 ** -23 * ref)
    assert bad_desc == 0 and bad_asc > 0

"""Pins the CPU checker's router functions (oracle/ferrule_oracle.c ``fo_router_*``) without a GPU:
against the literal vectors that Ferrule's own tests hold, against numpy's float64 routines and
stable lexsort, and against invariants; then the host-side validation that mirrors context.rs."""
import numpy as np
import pytest

from oracle import pyoracle as po


from oracle.parity import f64_scores  # noqa: E402


def ulp_distance(a32, b64):
    a32 = np.asarray(a32, np.float32)
    return np.abs(a32.astype(np.float64) - b64) / np.spacing(np.abs(b64).astype(np.float32)).astype(np.float64)


# ---- literal vectors of the reference's tests --------------------------------------------------

def test_reference_score_topk_order_and_weights():
    # routing.rs:378-391 sqrt_softplus_router_normalizes_and_scales_weights
    idx, w, s, _ = po.router_route_sqrt_softplus([0.0, 1.0, -1.0], 2, 1.5)
    assert idx.tolist() == [1, 0]
    want = f64_scores([1.0, 0.0])
    assert np.all(ulp_distance(s, want) <= 2)
    assert np.all(ulp_distance(w, want / want.sum() * 1.5) <= 4)
    # softplus(0) = ln 2 exactly
    assert abs(float(s[1]) - np.sqrt(np.log(2.0))) < 6e-8


def test_reference_bias_moves_selection_but_not_gathered_scores():
    # routing.rs:393-408 bias_changes_score_topk_selection_but_not_gathered_scores
    idx, _, s, sel = po.router_route_sqrt_softplus([5.0, 4.0, -4.0], 2, 1.0, bias=[0.0, 0.0, 10.0])
    assert idx.tolist() == [2, 0]
    assert ulp_distance(s[0], f64_scores([-4.0])[0]) <= 2
    assert ulp_distance(sel[0], f64_scores([-4.0])[0] + 10.0) <= 2


def test_reference_hash_router_keeps_table_order():
    # routing.rs:410-425 hash_router_preserves_hash_indices_and_gathers_original_scores
    idx, w, _, _ = po.router_route_sqrt_softplus([0.0, 1.0, 2.0], 2, 1.5, hash_experts=[2, 0])
    assert idx.tolist() == [2, 0]
    want = f64_scores([2.0, 0.0])
    assert np.all(ulp_distance(w, want / want.sum() * 1.5) <= 4)


HASH_LOGITS = np.array([[-2.0, 0.5, 3.0, -0.25], [2.0, -1.0, 0.0, 4.0], [1.0, 2.0, -3.0, 0.25]], np.float32)
HASH_TABLE = np.array([[3, 1, 2], [0, 2, 1], [1, 3, 0], [2, 0, 3], [0, 1, 2]], np.int32)
HASH_TOKENS = [3, 0, 3]
HASH_EXPECTED = [[2, 0], [3, 1], [2, 0]]   # dsv4_decode_topk_boundary.rs:757


def test_reference_device_hash_router_vector():
    # dsv4_decode_topk_boundary.rs:732-840: the expected ids are literal in the reference
    idx, w = po.router_kernel_rows(2, HASH_LOGITS, 2, 1.5, token_ids=HASH_TOKENS, hash_table=HASH_TABLE)
    assert idx.tolist() == HASH_EXPECTED
    for row in range(3):
        sc = f64_scores(HASH_LOGITS[row, HASH_EXPECTED[row]])
        assert np.all(np.abs(w[row] - sc / sc.sum() * 1.5) <= 1e-4)      # the reference's tolerance
        assert np.all(ulp_distance(w[row], sc / sc.sum() * 1.5) <= 4)    # ours


TOPK_LOGITS = np.array([[-2.0, 0.5, 3.0, -0.25, 1.5, -4.0], [2.0, -1.0, 0.0, 4.0, -3.0, 1.0]], np.float32)
TOPK_BIAS = np.array([0.0, 0.25, -0.5, 0.0, 0.75, -0.25], np.float32)


def test_reference_device_topk_router_case_against_float64_ranking():
    # dsv4_decode_topk_boundary.rs:629-690 (inputs literal there; the expectation is the ranking of
    # score + bias, done here in float64 with numpy's stable sort)
    idx, w = po.router_kernel_rows(1, TOPK_LOGITS, 3, 1.25, bias=TOPK_BIAS)
    for row in range(2):
        sc = f64_scores(TOPK_LOGITS[row])
        order = np.lexsort((np.arange(6), -(sc + TOPK_BIAS)))[:3]
        assert idx[row].tolist() == order.tolist()
        assert np.all(ulp_distance(w[row], sc[order] / sc[order].sum() * 1.25) <= 4)
    assert idx.tolist() == [[4, 2, 1], [3, 0, 4]]


# ---- library routines, brute force, invariants ---------------------------------------------------

def test_softplus_against_float64_over_the_branch_points():
    xs = np.concatenate([np.linspace(-104.0, 25.0, 5161), [-20.0, 20.0, np.nextafter(np.float32(20.0), np.float32(30.0)),
                                                           np.nextafter(np.float32(-20.0), np.float32(-30.0)), 0.0, -0.0]])
    xs = xs.astype(np.float32)
    got = np.array([po.stable_softplus(float(x)) for x in xs], np.float32)
    want = f64_scores(xs) ** 2
    normal = want > 1.2e-38
    assert np.all(ulp_distance(got[normal], want[normal]) <= 2)
    assert np.all(np.abs(got[~normal].astype(np.float64) - want[~normal]) <= 3e-45)
    assert np.all(got[xs > 20.0] == xs[xs > 20.0])


@pytest.mark.parametrize("experts,top_k,with_bias", [(256, 8, True), (256, 8, False), (64, 6, True), (384, 64, True),
                                                      (7, 7, False)])
def test_selection_equals_a_stable_sort_of_the_selection_scores(experts, top_k, with_bias):
    rng = np.random.default_rng(experts * 131 + top_k)
    for trial in range(40):
        logits = rng.normal(0.0, 2.0, experts).astype(np.float32)
        if trial % 4 == 0:
            logits[rng.integers(0, experts, experts // 2)] = logits[0]      # many exact ties
        bias = (rng.normal(0.0, 0.3, experts).astype(np.float32) if with_bias else None)
        idx, w, s, sel = po.router_route_sqrt_softplus(logits, top_k, 2.5, bias=bias)
        # all scores through the checker's own softplus, f32 sqrt and f32 add being correctly rounded
        scores = np.sqrt(np.array([po.stable_softplus(float(v)) for v in logits], np.float32))
        selection = scores + bias if with_bias else scores
        order = np.lexsort((np.arange(experts), -selection.astype(np.float64)))[:top_k]
        assert idx.tolist() == order.tolist()
        assert np.array_equal(s, scores[order]) and np.array_equal(sel, selection[order])
        # left-to-right f32 sum, one division, one multiplication
        total = np.float32(0.0)
        for v in scores[order]:
            total = np.float32(total + v)
        assert np.array_equal(w, (scores[order] / total * np.float32(2.5)).astype(np.float32))
        assert abs(float(w.astype(np.float64).sum()) - 2.5) < 2.5 * top_k * 2.0 ** -23


def test_device_restatement_equals_the_cpu_policy_on_finite_inputs():
    rng = np.random.default_rng(77)
    logits = rng.normal(0.0, 6.0, (96, 256)).astype(np.float32)
    logits[3, :40] = -30.0 - np.arange(40)          # the device's exp() branch below -20
    logits[4, :16] = 21.0 + np.arange(16)           # identity branch above 20
    bias = rng.normal(0.0, 0.2, 256).astype(np.float32)
    idx, w = po.router_kernel_rows(1, logits, 8, 2.5, bias=bias)
    for row in range(96):
        want_idx, want_w, _, _ = po.router_route_sqrt_softplus(logits[row], 8, 2.5, bias=bias)
        assert idx[row].tolist() == want_idx.tolist()
        assert np.array_equal(w[row], want_w)


def test_plain_topk_kinds_sort_values_and_break_ties_by_column():
    rng = np.random.default_rng(5)
    logits = rng.integers(-4, 5, (32, 150)).astype(np.float32)       # heavy ties
    logits[0, 10] = -0.0
    logits[0, 3] = 0.0
    idx, val = po.router_kernel_rows(4, logits, 40)
    idx_f, val_f = po.router_kernel_rows(3, logits, 40)
    for row in range(32):
        order = np.lexsort((np.arange(150), -logits[row].astype(np.float64)))[:40]
        assert idx[row].tolist() == order.tolist()
        assert np.array_equal(val[row], logits[row, order])
    assert idx_f.dtype == np.float32 and np.array_equal(idx_f, idx.astype(np.float32)) and np.array_equal(val_f, val)


def test_more_slots_than_columns_and_untouched_rows():
    idx, w = po.router_kernel_rows(1, np.array([[0.0, 1.0, -1.0]], np.float32), 5, 1.0)
    assert idx.tolist() == [[1, 0, 2, -1, -1]] and w[0, 3] == 0.0 and w[0, 4] == 0.0
    idx4, val4 = po.router_kernel_rows(4, np.array([[0.0, 1.0, -1.0]], np.float32), 5)
    assert idx4.tolist() == [[1, 0, 2, -1, -1]] and np.isneginf(val4[0, 3:]).all()
    # a token id outside the table, or a table entry outside the experts, leaves the row as it was
    table = HASH_TABLE.copy()
    table[0, 1] = 9
    before_i = np.full((3, 2), 77, np.int32)
    before_w = np.full((3, 2), 0.5, np.float32)
    idx, w = po.router_kernel_rows(2, HASH_LOGITS, 2, 1.5, token_ids=[3, 0, 5], hash_table=table, indices=before_i,
                                   weights=before_w)
    assert idx.tolist() == [[2, 0], [77, 77], [77, 77]] and w[1:].tolist() == [[0.5, 0.5], [0.5, 0.5]]
    # the k range the kernel accepts: outside it nothing is written
    idx, w = po.router_kernel_rows(4, HASH_LOGITS, 65, indices=np.full((3, 65), 9, np.int32))
    assert (idx == 9).all()


def test_policy_validation_follows_the_reference():
    # routing.rs:209-289
    with pytest.raises(po.OracleError):
        po.router_route_sqrt_softplus([0.0, 1.0], 3, 1.0)
    with pytest.raises(po.OracleError):
        po.router_route_sqrt_softplus([0.0, np.inf], 1, 1.0)
    with pytest.raises(po.OracleError):
        po.router_route_sqrt_softplus([0.0, 1.0], 1, np.nan)
    with pytest.raises(po.OracleError):
        po.router_route_sqrt_softplus([0.0, 1.0], 1, 1.0, bias=[0.0, np.nan])
    with pytest.raises(po.OracleError):
        po.router_route_sqrt_softplus([0.0, 1.0, 2.0], 2, 1.0, hash_experts=[1, 1])
    with pytest.raises(po.OracleError):
        po.router_route_sqrt_softplus([0.0, 1.0, 2.0], 2, 1.0, hash_experts=[3, 1])
    with pytest.raises(po.OracleError):
        po.router_route_sqrt_softplus([0.0, 1.0, 2.0], 2, 1.0, hash_experts=[1])
    # every score underflows to zero: "non-positive weight sum"
    with pytest.raises(po.OracleError):
        po.router_route_sqrt_softplus([-200.0, -200.0], 1, 1.0)


def test_host_validation_of_token_ids_and_hash_tables():
    # dsv4_decode_topk_boundary.rs:692-729
    from ferrule_amd.provider import validate_dsv4_router_hash_table, validate_dsv4_router_token_ids

    assert validate_dsv4_router_token_ids([2, 0], 3) == [2, 0]
    with pytest.raises(ValueError, match="batch row 0"):
        validate_dsv4_router_token_ids([3], 3)
    valid = [0, 1, 2, 2, 0, 1]
    assert validate_dsv4_router_hash_table(valid, 2, 3, 3, 2) == valid
    with pytest.raises(ValueError, match="top_k"):
        validate_dsv4_router_hash_table(valid, 2, 3, 3, 4)
    with pytest.raises(ValueError, match="duplicate expert id 1"):
        validate_dsv4_router_hash_table([1, 1, 0], 1, 3, 3, 2)
    with pytest.raises(ValueError, match="exceeds expert count 3"):
        validate_dsv4_router_hash_table([3, 1, 0], 1, 3, 3, 2)


def test_router_launch_validation_codes_without_touching_a_device():
    from ferrule_amd import abi
    import ctypes as C

    lib = abi.load()
    assert lib.ferrule_hip_core_router_launch(None) == 1
    base = dict(kind=abi.ROUTER_TOPK, rows=4, columns=16, k=2, route_scale=1.0, logits=0x1000, indices=0x2000,
                weights=0x3000)
    for change in (dict(kind=0), dict(kind=5), dict(logits=0), dict(indices=0), dict(weights=0),
                   dict(flags=1, bias=0), dict(kind=abi.ROUTER_HASH), dict(kind=abi.ROUTER_HASH, token_ids=0x10,
                                                                         hash_table=0x20, hash_columns=1)):
        args = abi.RouterArgs(**{**base, **change})
        assert lib.ferrule_hip_core_router_launch(C.byref(args)) == 1, change
    # shapes for which the reference kernel returns at once: success, nothing launched
    for change in (dict(k=0), dict(k=65), dict(rows=0)):
        args = abi.RouterArgs(**{**base, **change})
        assert lib.ferrule_hip_core_router_launch(C.byref(args)) == 0, change

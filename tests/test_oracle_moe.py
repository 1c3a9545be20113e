"""Pins the routed-FFN oracle: brute force on tiny shapes, the C restatement, permutation
invariance, the torch-op variant, and the seed-0 routing histogram of the benchmark config."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import moe_ffn, mxfp8

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _small_case(seed=0, T=40, H=64, I=96, E=3, k=2, empty=None):
    rng = np.random.default_rng(seed)
    logits = torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32))
    if empty is not None:
        logits[:, empty] = -1e9
    idx = moe_ffn.route_topk(logits, k).numpy()
    counts, row_token, _ = moe_ffn.group_rows(idx, E)
    x_q, x_sc = mxfp8.mx_quantize(rng.standard_normal((T, H)).astype(np.float32))
    w = lambda n, kk: mxfp8.mx_quantize((rng.standard_normal((E, n, kk)) * 0.2).astype(np.float32))
    (wg_q, wg_sc), (wu_q, wu_sc), (wd_q, wd_sc) = w(I, H), w(I, H), w(H, I)
    return dict(x_q=x_q, x_sc=x_sc, wg_q=wg_q, wg_sc=wg_sc, wu_q=wu_q, wu_sc=wu_sc, wd_q=wd_q, wd_sc=wd_sc,
                counts=counts, row_token=row_token)


def test_grouped_matmul_vs_triple_loop_with_empty_and_single_row_experts():
    rng = np.random.default_rng(5)
    counts = np.array([0, 1, 33], dtype=np.int32)
    a = rng.standard_normal((34, 64)).astype(np.float32)
    w = rng.standard_normal((3, 32, 64)).astype(np.float32)
    fast = moe_ffn.grouped_matmul(a, w, counts)
    slow = moe_ffn.grouped_matmul_naive(a, w, counts)
    assert np.allclose(fast, slow, rtol=1e-5, atol=1e-5)
    assert np.allclose(fast[0], a[0] @ w[1].T, rtol=1e-5, atol=1e-5)  # the single row of expert 1


def test_topk_of_softmax_is_topk_of_logits_and_counts_sum():
    logits = torch.randn(500, 32, generator=torch.Generator().manual_seed(7))
    idx = moe_ffn.route_topk(logits, 4)
    assert torch.equal(idx, torch.topk(logits, 4, dim=-1).indices)
    counts, row_token, row_slot = moe_ffn.group_rows(idx.numpy(), 32)
    assert counts.sum() == 2000 and len(row_token) == 2000
    experts = idx.numpy()[row_token, row_slot]
    assert np.all(np.diff(experts) >= 0)                       # grouped by expert
    for e in range(32):                                        # stable: token order kept inside an expert
        assert np.all(np.diff(row_token[experts == e]) >= 0)


def test_forward_matches_c_restatement(c_oracle):
    case = _small_case(seed=1, empty=1)
    assert case["counts"][1] == 0
    ref = moe_ffn.moe_ffn_forward(**case)
    R, H, I = len(case["row_token"]), 64, 96
    y = np.zeros((R, H), np.float32)
    hq = np.zeros((R, I), np.uint8)
    hsc = np.zeros((R, case["wd_sc"].shape[-1]), np.uint8)
    arrs = [np.ascontiguousarray(case[k]) for k in ("x_q", "x_sc", "row_token", "wg_q", "wg_sc", "wu_q", "wu_sc",
                                                     "wd_q", "wd_sc", "counts")]
    c_oracle.plko_moe_forward(*[a.ctypes.data for a in arrs], 3, H, I, case["x_sc"].shape[-1], hsc.shape[-1], 7.0, 1,
                              y.ctypes.data, hq.ctypes.data, hsc.ctypes.data)
    # accumulation order differs (float64 scalar loop vs BLAS fp32): hidden may flip a bf16 ulp, so compare values
    hid_c = mxfp8.mx_dequantize(hq, hsc)
    hid_n = mxfp8.mx_dequantize(ref["hidden_q"], ref["hidden_sc"])
    assert moe_ffn.rel_frobenius(hid_c, hid_n) < 2e-3
    assert (hq != ref["hidden_q"]).mean() < 0.02
    assert moe_ffn.rel_frobenius(y, ref["y"]) < 5e-3


def test_forward_token_permutation_permutes_rows():
    case = _small_case(seed=2)
    ref = moe_ffn.moe_ffn_forward(**case)
    perm = np.random.default_rng(0).permutation(case["x_q"].shape[0])
    inv = np.argsort(perm)
    case2 = dict(case, x_q=case["x_q"][perm], x_sc=case["x_sc"][perm], row_token=inv[case["row_token"]].astype(np.int32))
    out = moe_ffn.moe_ffn_forward(**case2)
    assert np.array_equal(out["y_bf16_bits"], ref["y_bf16_bits"])


def test_torch_variant_agrees_with_numpy_oracle():
    case = _small_case(seed=3, T=64, H=128, I=160, E=4)
    ref = moe_ffn.moe_ffn_forward(**case)
    t = {k: torch.from_numpy(np.ascontiguousarray(v)) for k, v in case.items()}
    y = moe_ffn.moe_ffn_forward_torch(**t).float().numpy()
    assert moe_ffn.rel_frobenius(y, ref["y"]) < 2e-3


def test_hidden_is_bf16_before_requant_and_quantised_blocks_are_consistent():
    case = _small_case(seed=4)
    ref = moe_ffn.moe_ffn_forward(**case)
    assert np.array_equal(mxfp8.bf16_round(ref["hidden"]), ref["hidden"])
    q2, sc2 = mxfp8.mx_quantize(ref["hidden"])
    assert np.array_equal(q2, ref["hidden_q"]) and np.array_equal(sc2, ref["hidden_sc"])


def test_seed0_routing_histogram_fixture():
    """tokens_per_expert of the benchmark config (T=8192, E=32, top-4, seed 0) is pinned as a fixture."""
    logits = torch.randn(8192, 32, generator=torch.Generator().manual_seed(0))
    counts, row_token, _ = moe_ffn.group_rows(moe_ffn.route_topk(logits, 4).numpy(), 32)
    with open(os.path.join(GOLDEN, "routing_seed0_T8192_E32_top4.json")) as fh:
        want = json.load(fh)
    assert counts.tolist() == want["tokens_per_expert"]
    assert int(row_token[:8].sum()) == want["row_token_first8_sum"] and counts.sum() == 32768


def test_harness_error_reports_follow_their_definitions():
    from pipelink_amd.host import mok_inputs

    ref = np.array([[1.0, -2.0], [4.0, 0.0]], dtype=np.float32)
    got = np.array([[1.5, -2.0], [3.0, 0.25]], dtype=np.float32)
    mean, maximum, relative = mok_inputs.error_stats(ref, got)
    assert mean == pytest.approx((0.5 + 0 + 1.0 + 0.25) / 4) and maximum == 1.0
    assert relative == pytest.approx(1.75 / 7.0)
    assert mok_inputs.error_stats(ref, got, chunk=3) == pytest.approx((mean, maximum, relative))   # chunking changes nothing
    rep = mok_inputs.tolerance_report(ref, got)
    assert rep["passed"] is False and rep["abs_max"] == 1.0 and rep["relative_tolerance"] == 1e-2   # 1.0 > 5e-1
    assert mok_inputs.tolerance_report(ref, ref)["passed"] is True
    assert mok_inputs.tolerance_report(ref, np.full_like(ref, np.nan))["passed"] is False           # NaN never passes
    assert mok_inputs.error_stats(np.zeros(3), np.zeros(3)) == (0.0, 0.0, 0.0)
    a = torch.arange(6, dtype=torch.bfloat16).reshape(2, 3)
    assert mok_inputs.bitwise_report(a, a.clone()) and not mok_inputs.bitwise_report(a, a + 1)
    assert not mok_inputs.bitwise_report(a, a.reshape(3, 2).t())                                     # same values, other layout
    assert mok_inputs.bitwise_report(np.float32([0.0]), np.float32([0.0])) and not mok_inputs.bitwise_report(np.float32([0.0]), np.float32([-0.0]))

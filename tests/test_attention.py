"""Flash-attention prefill stage (core + swappable mask package) and the output projection after it.

CPU part: the oracle's pins and what the link records.  GPU part (marked gpu): a small case against the
oracle on every head; the stated case -- bf16, batch 4, 32 query / 8 KV heads, head dimension 128, 4096
tokens, causal -- on sampled heads, linked image byte-identical to the one-unit control, and the output
projection (the bf16 GEMM packages of the one-epilogue example, W_o from N(0,1) * 0.02) on sampled rows."""
import json
import shutil
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import attention as oa
from pipelink_amd.stages.attention import build as fa_build

ROOT = Path(__file__).resolve().parents[1]
needs_rocm = pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(),
                                reason="needs the ROCm toolchain")


def test_oracle_against_the_library_and_closed_forms():
    q, k, v = oa.inputs(1, 2, 1, 96, seed=1)
    mine = oa.attention_head(q[0, 1], k[0, 0], v[0, 0])
    lib = oa.attention_head_library(q[0, 1], k[0, 0], v[0, 0])
    assert torch.allclose(mine, lib, rtol=1e-5, atol=1e-6)
    assert torch.allclose(mine[0], v[0, 0, 0].float())                      # the first query sees only key 0
    same_k = k[0, 0, :1].expand(96, 128)
    mean = oa.attention_head(q[0, 0], same_k, v[0, 0])
    running = v[0, 0].float().cumsum(0) / torch.arange(1, 97)[:, None]
    assert torch.allclose(mean, running, rtol=1e-5, atol=1e-6)              # equal scores: a running mean of V
    heads = oa.attention(q, k, v)
    assert set(heads) == {(0, 0), (0, 1)} and torch.equal(heads[(0, 1)], mine)   # both query heads read KV head 0
    # sliding window: one key -> the query's own V row; a window as long as the sequence -> plain causal; equal
    # scores -> the mean of the last `window` rows of V
    assert torch.allclose(oa.attention_head(q[0, 1], k[0, 0], v[0, 0], window=1), v[0, 0].float())
    assert torch.equal(oa.attention_head(q[0, 1], k[0, 0], v[0, 0], window=96), mine)
    vf = v[0, 0].float()
    sums = vf.cumsum(0)
    sums[5:] -= vf.cumsum(0)[:-5].clone()
    last5 = sums / torch.arange(1, 97).clamp(max=5)[:, None]
    assert torch.allclose(oa.attention_head(q[0, 0], same_k, v[0, 0], window=5), last5, rtol=1e-4, atol=1e-5)


@pytest.fixture(scope="module")
def example(tmp_path_factory):
    out = tmp_path_factory.mktemp("attention")
    return out, fa_build.build(out=out, one_unit=False)


@needs_rocm
def test_link_records_core_and_mask_packages(example):
    out, res = example
    link = res["link"]
    assert [e["stage_id"] for e in link["params"]["entries"]] == ["fa.core", "fa.mask.causal"]
    assert [(e["offset"], e["bytes"]) for e in link["params"]["entries"]] == [(0, 56), (56, 8)]
    assert link["threads"] == 256 and link["dyn_smem_bytes"] == 2 * 2 * 64 * 256 == 65536
    assert {e["channel"] for e in link["protocol_expansions"]} == {"mask_key_count", "mask_key_begin", "mask_all_visible", "mask_visible"}
    obs = link["observed"]
    assert obs["calls"] == 0 and obs["mfma"] == 64 and obs["private_segment_fixed_size"] == 0   # the mask is inlined; the block loop is unrolled by two
    from pipelink_amd.stages.attention.params import params_blobs
    blobs = params_blobs({"q": 1, "k": 2, "v": 3, "o": 4}, 4, 32, 8, 4096)
    assert {sid: len(b) for sid, b in blobs.items()} == {"fa.core": 56, "fa.mask.causal": 8}


@needs_rocm
def test_window_mask_is_a_relink_of_the_same_core_package(example):
    out, res = example
    link, window = res["link"], res["window"]
    assert [e["stage_id"] for e in window["params"]["entries"]] == ["fa.core", "fa.mask.window"]
    assert window["input_hashes"]["fa.core"] == link["input_hashes"]["fa.core"]   # the same package bytes went into both links
    assert set(window["input_hashes"]) == {"fa.core", "fa.mask.window"}
    assert window["observed"]["calls"] == 0 and window["observed"]["mfma"] == 64
    from pipelink_amd.stages.attention.params import params_blobs
    blobs = params_blobs({"q": 1, "k": 2, "v": 3, "o": 4}, 4, 32, 8, 4096, window=1024)
    assert set(blobs) == {"fa.core", "fa.mask.window"} and blobs["fa.mask.window"] == (4096).to_bytes(4, "little") + (1024).to_bytes(4, "little")


def test_host_rejects_shapes_the_kernel_does_not_handle():
    from pipelink_amd.host.attention import open_session

    z = lambda *s: np.zeros(s, dtype=np.uint16)
    for q, k in ((z(1, 4, 100, 128), z(1, 2, 100, 128)), (z(1, 4, 128, 64), z(1, 2, 128, 64)), (z(1, 3, 128, 128), z(1, 2, 128, 128))):
        with pytest.raises(ValueError):
            open_session("unused.json", q, k, k)


# ---- GPU ---------------------------------------------------------------------------------------------------

def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16).float()


def _check_heads(o: torch.Tensor, q, k, v, heads):
    """o [B, S, Hq*D] fp32 against the oracle on the listed heads: bf16 output rounding + bf16 probabilities."""
    ref = oa.attention(q, k, v, heads)
    for (b, h), want in ref.items():
        got = o[b, :, h * 128:(h + 1) * 128]
        assert torch.isfinite(got).all()
        err = (got - want).abs().max().item()
        assert err <= 1e-2 * want.abs().max().item(), (b, h, err)
        assert ((got - want).norm() / want.norm()).item() <= 1e-2, (b, h)


@pytest.mark.gpu
def test_small_case_matches_the_oracle_on_every_head():
    from pipelink_amd.host.attention import open_session

    paths = fa_build.images()
    q, k, v = oa.inputs(2, 4, 2, 384, seed=3)
    sess = open_session(paths["link_json"], _bits(q), _bits(k), _bits(v))
    try:
        sess.write("o", np.full((2, 384, 512), 0x7FC0, dtype=np.uint16))
        sess.launch()
        sess.synchronize()
        o = _from_bits(sess.read("o"))
    finally:
        sess.close()
    _check_heads(o, q, k, v, None)


@pytest.mark.gpu
@pytest.mark.parametrize("window", [1, 100, 128, 300, 4096])
def test_window_mask_matches_the_oracle_on_every_head(window):
    """The relinked image (fa.core + fa.mask.window): windows below, at and above the 64-key block and the 128-query
    tile, and one longer than the sequence (plain causal)."""
    from pipelink_amd.host.attention import open_session

    paths = fa_build.images()
    q, k, v = oa.inputs(1, 4, 2, 640, seed=5)
    sess = open_session(paths["window_link_json"], _bits(q), _bits(k), _bits(v), window=window)
    try:
        sess.write("o", np.full((1, 640, 512), 0x7FC0, dtype=np.uint16))
        sess.launch()
        sess.synchronize()
        o = _from_bits(sess.read("o"))
    finally:
        sess.close()
    ref = oa.attention(q, k, v, None, window=window)
    for (b, h), want in ref.items():
        got = o[b, :, h * 128:(h + 1) * 128]
        assert torch.isfinite(got).all()
        assert (got - want).abs().max().item() <= 1e-2 * want.abs().max().item(), (b, h)
        assert ((got - want).norm() / want.norm()).item() <= 1e-2, (b, h)


@pytest.mark.gpu
def test_window_mask_with_a_small_softmax_scale():
    """A caller's scale far below 1 / sqrt(128): queries whose first streamed block holds no key they may see must
    still give that block zero weight (whether a query has seen a key is decided on unscaled scores)."""
    from pipelink_amd.host.attention import open_session

    paths = fa_build.images()
    q, k, v = oa.inputs(1, 4, 2, 640, seed=9)
    scale = 2.0 ** -10
    sess = open_session(paths["window_link_json"], _bits(q), _bits(k), _bits(v), window=100, scale=scale)
    try:
        sess.write("o", np.full((1, 640, 512), 0x7FC0, dtype=np.uint16))
        sess.launch()
        sess.synchronize()
        o = _from_bits(sess.read("o"))
    finally:
        sess.close()
    for h in range(4):
        want = oa.attention_head(q[0, h], k[0, h // 2], v[0, h // 2], scale=scale, window=100)
        got = o[0, :, h * 128:(h + 1) * 128]
        assert torch.isfinite(got).all()
        assert (got - want).abs().max().item() <= 1e-2 * want.abs().max().item(), h
        assert ((got - want).norm() / want.norm()).item() <= 1e-2, h


def test_the_host_rejects_a_scale_that_is_not_positive_and_finite():
    from pipelink_amd.host.attention import open_session

    q = np.zeros((1, 2, 128, 128), dtype=np.uint16)
    kv = np.zeros((1, 1, 128, 128), dtype=np.uint16)
    for bad in (0.0, -0.1, float("inf"), float("nan")):
        with pytest.raises(ValueError, match="scale"):
            open_session("unused.json", q, kv, kv, scale=bad)


@pytest.mark.gpu
def test_window_mask_at_the_stated_size_on_sampled_heads():
    """B 4, 32 / 8 heads, S 4096 with a window of 1024 keys: tiles start streaming at their first visible block."""
    from pipelink_amd.host.attention import open_session

    B, HQ, HKV, S, W = 4, 32, 8, 4096, 1024
    q, k, v = oa.inputs(B, HQ, HKV, S, seed=0)
    sess = open_session(fa_build.images()["window_link_json"], _bits(q), _bits(k), _bits(v), window=W)
    try:
        sess.write("o", np.full((B, S, HQ * 128), 0x7FC0, dtype=np.uint16))
        sess.launch()
        sess.synchronize()
        o = _from_bits(sess.read("o"))
        ms = sorted(sess.time(50) for _ in range(3))[1]
        print(f"attention, window {W}: {ms:.3f} ms", flush=True)
    finally:
        sess.close()
    for (b, h), want in oa.attention(q, k, v, [(0, 5), (2, 17)], window=W).items():
        got = o[b, :, h * 128:(h + 1) * 128]
        assert torch.isfinite(got).all()
        assert (got - want).abs().max().item() <= 1e-2 * want.abs().max().item(), (b, h)
        assert ((got - want).norm() / want.norm()).item() <= 1e-2, (b, h)


@pytest.mark.gpu
def test_stated_case_sampled_heads_one_unit_control_and_output_projection():
    from pipelink_amd.host.attention import open_session
    from pipelink_amd.host.one_epilogue import open_session as open_gemm
    from pipelink_amd.stages.one_epilogue import build as oe_build

    B, HQ, HKV, S = 4, 32, 8, 4096
    q, k, v = oa.inputs(B, HQ, HKV, S, seed=0)
    paths = fa_build.images()
    sess = open_session(paths["link_json"], _bits(q), _bits(k), _bits(v))
    try:
        sess.write("o", np.full((B, S, HQ * 128), 0x7FC0, dtype=np.uint16))
        sess.launch()
        sess.synchronize()
        o_bits = sess.read("o")
        control = sess.with_image(paths["one_unit"])
        sess.write("o", np.full((B, S, HQ * 128), 0x7FC0, dtype=np.uint16))
        control.launch()
        control.synchronize()
        assert np.array_equal(sess.read("o"), o_bits), "linked and one-unit images differ"
        import time
        start = time.time()
        while time.time() - start < 1.0:     # the GPU needs about a second of load to reach its sustained clock state
            sess.time(50)
        ms = sorted(sess.time(100) for _ in range(3))[1]
        print(f"attention: {ms:.3f} ms sustained, {4 * B * HQ * S * S * 128 / 2 / ms / 1e9:.0f} TFLOP/s on causal flop", flush=True)
    finally:
        sess.close()
    o = _from_bits(o_bits)
    _check_heads(o, q, k, v, [(0, 0), (1, 13), (3, 31)])
    # output projection: y = O . W_o^T, W_o [4096, 4096] from N(0,1) * 0.02, through the linked bf16 GEMM
    g = torch.Generator().manual_seed(1)
    w_o = (torch.randn(HQ * 128, HQ * 128, generator=g) * 0.02).to(torch.bfloat16)     # [out, in]: already "B^T"
    gemm = oe_build.images("full")     # the 256 x 256 tile
    ones, zeros = np.ones(HQ * 128, dtype=np.float32), np.zeros(HQ * 128, dtype=np.float32)
    proj = open_gemm(gemm["link_json"], "full", o_bits.reshape(B * S, HQ * 128), _bits(w_o), zeros, ones)
    try:
        proj.launch()
        proj.synchronize()
        assert proj.read("status")[0] == 0
        y = _from_bits(proj.read("c"))
        pms = sorted(proj.time(20) for _ in range(3))[1]
        print(f"output projection: {pms:.3f} ms, {2 * B * S * (HQ * 128) ** 2 / pms / 1e9:.0f} TFLOP/s", flush=True)
    finally:
        proj.close()
    rows = torch.from_numpy(np.random.default_rng(0).choice(B * S, 32, replace=False))
    want = (o.reshape(B * S, -1)[rows] @ w_o.float().t()).to(torch.bfloat16).float()
    got = y[rows]
    assert ((got - want).abs().max() / want.abs().max()).item() <= 1e-2
    assert ((got - want).norm() / want.norm()).item() <= 3e-3

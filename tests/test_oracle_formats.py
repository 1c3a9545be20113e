"""Pins the oracle's number formats and quantiser against independent evidence:
torch's float8 dtypes (library routines), the C restatement, closed forms and invariants."""
import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from oracle import mxfp8


def _all_bf16_as_f32():
    return (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)


def test_e4m3_decode_matches_torch_view():
    codes = np.arange(256, dtype=np.uint8)
    ours = mxfp8.e4m3_decode(codes)
    theirs = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(ours), np.isnan(theirs))
    m = ~np.isnan(ours)
    assert np.array_equal(ours[m], theirs[m])
    assert ours[0x7E] == 448.0 and ours[0x01] == 2.0 ** -9 and ours[0x08] == 2.0 ** -6


def test_e4m3_decode_matches_c(c_oracle):
    for c in range(256):
        a, b = float(mxfp8.e4m3_decode(np.uint8(c))), c_oracle.plko_e4m3_decode(c)
        assert (np.isnan(a) and np.isnan(b)) or a == b


def test_e4m3_encode_all_bf16_vs_torch_clamped():
    x = _all_bf16_as_f32()
    x = x[np.isfinite(x)]
    ours = mxfp8.e4m3_encode(x)
    clamped = torch.from_numpy(x).clamp(-448.0, 448.0)
    theirs = clamped.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    # -0.0 vs +0.0: both are zeros; compare sign bit too (torch keeps the sign)
    assert np.array_equal(ours, theirs)


def test_e4m3_encode_dense_fp32_sweep_vs_torch():
    rng = np.random.default_rng(1)
    # log-uniform magnitudes across and beyond the representable range, plus exact ties
    mags = np.exp2(rng.uniform(-12, 10, size=200000)).astype(np.float32)
    x = mags * rng.choice(np.float32([-1, 1]), size=mags.shape)
    ties = (mxfp8.e4m3_decode(np.arange(0, 0x7E, dtype=np.uint8)) +
            mxfp8.e4m3_decode(np.arange(1, 0x7F, dtype=np.uint8))) / 2
    x = np.concatenate([x, ties.astype(np.float32), -ties.astype(np.float32)])
    ours = mxfp8.e4m3_encode(x)
    theirs = torch.from_numpy(x).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(ours, theirs)


def test_e4m3_encode_matches_c(c_oracle):
    rng = np.random.default_rng(2)
    x = np.concatenate([
        (np.exp2(rng.uniform(-12, 10, size=20000)) * rng.choice([-1, 1], size=20000)).astype(np.float32),
        np.float32([0.0, -0.0, 448, 449, 464, 465, 480, 1e9, -1e9, 2 ** -10, 2 ** -9, 3 * 2 ** -10, 2 ** -6]),
    ])
    ours = mxfp8.e4m3_encode(x)
    theirs = np.array([c_oracle.plko_e4m3_encode(float(v)) for v in x], dtype=np.uint8)
    assert np.array_equal(ours, theirs)


def test_e4m3_encode_known_answers():
    x = np.float32([448, 449, 464, 465, 1000, np.inf, -1e9, 2 ** -10, 2 ** -9, 3 * 2 ** -10, 1.0, 1.0625, 1.1875])
    # 2**-10 ties to even (0); 3*2**-10 = 1.5 ulp ties to even (2); 1.0625 ties to 1.0; 1.1875 ties to 1.25
    assert mxfp8.e4m3_encode(x).tolist() == [126, 126, 126, 126, 126, 126, 254, 0, 1, 2, 0x38, 0x38, 0x3A]
    assert mxfp8.e4m3_encode(np.float32([np.nan]))[0] & 0x7F == 0x7F


def test_e4m3_roundtrip_exact_for_every_code():
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    assert np.array_equal(mxfp8.e4m3_encode(mxfp8.e4m3_decode(codes)), codes)


def test_e8m0_matches_torch_and_closed_form(c_oracle):
    b = np.arange(0, 255, dtype=np.uint8)
    ours = mxfp8.e8m0_decode(b)
    theirs = torch.from_numpy(b).view(torch.float8_e8m0fnu).float().numpy()
    assert np.array_equal(ours, theirs)
    assert ours[127] == 1.0 and ours[128] == 2.0 and ours[126] == 0.5
    assert np.isnan(mxfp8.e8m0_decode(np.uint8(255)))
    for v in [0.0, 1e-45, 1.0, 1.5, 2.0, 255.9, 256.0, 448.0, 3e38, 6e-39]:
        assert int(mxfp8.e8m0_from_amax(np.float32(v))) == c_oracle.plko_e8m0_from_amax(v)
    assert int(mxfp8.e8m0_from_amax(np.float32(256.0))) == 127
    assert int(mxfp8.e8m0_from_amax(np.float32(255.99))) == 126
    assert int(mxfp8.e8m0_from_amax(np.float32(1.0))) == 119


def test_bf16_round_matches_torch_and_c(c_oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal(100000).astype(np.float32) * np.exp2(rng.integers(-20, 20, 100000)).astype(np.float32)
    ours = mxfp8.bf16_round(x)
    theirs = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(ours, theirs)
    for v in x[:2000]:
        assert c_oracle.plko_bf16_round(float(v)) == float(mxfp8.bf16_round(np.float32([v]))[0])
    bits = mxfp8.bf16_bits(x)
    assert np.array_equal(bits, torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))


def test_mx_quantize_matches_c(c_oracle):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((37, 96)) * np.exp2(rng.integers(-30, 30, (37, 1)))).astype(np.float32)
    x[3] = 0.0
    x[5, :32] = 0.0
    q, sc = mxfp8.mx_quantize(x)
    ld = sc.shape[1]
    assert ld == 4
    cq = np.zeros_like(q)
    csc = np.zeros_like(sc)
    c_oracle.plko_mx_quantize(x.ctypes.data, 37, 96, ld, cq.ctypes.data, csc.ctypes.data)
    assert np.array_equal(q, cq) and np.array_equal(sc, csc)
    assert sc[3].tolist() == [0, 0, 0, 0] and not q[3].any()


@settings(max_examples=200, deadline=None)
@given(st.integers(0, 2 ** 32 - 1), st.integers(-100, 100))
def test_mx_quantize_invariants(seed, exp):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((4, 64)) * 2.0 ** exp).astype(np.float32)
    q, sc = mxfp8.mx_quantize(x)
    scale = mxfp8.e8m0_decode(sc[:, :2])
    # scale is an exact power of two
    m, _ = np.frexp(scale.astype(np.float64))
    assert np.all(m == 0.5)
    blk = np.abs(x.reshape(4, 2, 32))
    amax = blk.max(-1)
    normal = amax >= np.float32(2.0 ** -126) * 256  # blocks whose scale byte is not clamped at 0
    scaled = amax.astype(np.float64) / scale.astype(np.float64)
    assert np.all((scaled[normal] >= 256) & (scaled[normal] < 512))
    codes_max = np.abs(mxfp8.e4m3_decode(q)).reshape(4, 2, 32).max(-1)
    assert np.all((codes_max[normal] >= 256) & (codes_max[normal] <= 448))
    # relative error of unsaturated normal elements <= 2**-4
    d = mxfp8.mx_dequantize(q, sc)
    s = np.abs(x.reshape(4, 2, 32)).astype(np.float64) / scale[..., None].astype(np.float64)
    ok = (s >= 2.0 ** -6) & (s <= 448) & normal[..., None]
    err = np.abs(d.astype(np.float64) - x.astype(np.float64)).reshape(4, 2, 32)
    assert np.all(err[ok] <= np.abs(x.reshape(4, 2, 32))[ok].astype(np.float64) * 2.0 ** -4)
    # idempotence and sign symmetry
    q2, sc2 = mxfp8.mx_quantize(d)
    assert np.array_equal(q2, q) and np.array_equal(sc2[:, :2], sc[:, :2])
    qn, scn = mxfp8.mx_quantize(-x)
    assert np.array_equal(scn, sc) and np.array_equal(qn ^ 0x80, q)


def test_swiglu_special_values(c_oracle):
    from oracle.moe_ffn import gptoss_swiglu
    L = 7.0
    f = lambda g, u: float(gptoss_swiglu(np.float32([g]), np.float32([u]), L)[0])
    assert f(0.0, 3.0) == 0.0
    assert f(2.0, -1.0) == 0.0
    assert abs(f(-1e4, 2.0)) == 0.0
    assert f(100.0, 0.5) == f(7.0, 0.5)
    assert f(1.0, 100.0) == f(1.0, 7.0) and f(1.0, -100.0) == f(1.0, -7.0)
    sig = 1.0 / (1.0 + np.exp(-1.702 * 1.5))
    assert abs(f(1.5, 0.25) - 1.25 * 1.5 * sig) < 1e-6
    # unclamped variant
    assert float(gptoss_swiglu(np.float32([100.0]), np.float32([0.0]), None)[0]) == pytest.approx(100.0)
    for g, u in [(0.3, -2.0), (9.0, 9.0), (-3.0, 0.1)]:
        assert c_oracle.plko_swiglu(g, u, L, 1) == pytest.approx(f(g, u), rel=1e-6, abs=1e-7)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_host_quantiser_equals_the_oracle_bit_for_bit(dtype):
    """pipelink_amd.mxfp8.quantize (torch; what the harness-side code calls where the reference calls ops.mxfp8_quantize,
    campaigns/mok/host/mok_port_host.py:122) against oracle.mxfp8.mx_quantize: codes and scale bytes, on random data
    over 60 binades, blocks of zeros, blocks whose scale sits at 2^+-30, values that saturate after scaling only by
    rounding, subnormal inputs, NaN of both signs and infinities."""
    import torch
    from pipelink_amd import mxfp8 as host

    g = torch.Generator().manual_seed(11)
    x = torch.randn(64, 256, generator=g) * torch.exp2(torch.randint(-30, 31, (64, 8), generator=g).float()).repeat_interleave(32, dim=1)
    x[0] = 0                                   # a row of zero blocks: scale byte 0, codes 0
    x[1, :32] = 0
    x[2, :32] = torch.randn(32, generator=g) * 2.0 ** 30
    x[3, :32] = torch.randn(32, generator=g) * 2.0 ** -30
    x[4, :32] = 2.0 ** -130                    # fp32 subnormals: exponent field 0, scale byte 0
    x[5, 0], x[5, 1:32] = 1.99999, 0.001       # amax just below a power of two: the largest quotient rounds up to 256
    x[6, 0], x[6, 1] = 255.99, 447.9           # near the top of the e4m3 range before scaling
    x[7, 3] = float("nan")
    x[8, 40] = float("nan")
    x.view(torch.int32)[8, 40] |= -0x80000000  # NaN with the sign bit set
    x[9, 5], x[9, 70] = float("inf"), -float("inf")
    src = x.to(getattr(torch, dtype))
    q, sc = host.quantize(src)
    oq, osc = mxfp8.mx_quantize(src.float().numpy())
    assert np.array_equal(q.numpy(), oq)
    assert np.array_equal(sc.numpy()[:, :8], osc[:, :8]) and not sc.numpy()[:, 8:].any()
    assert not oq[0].any() and not osc[0].any() and oq[7, 3] & 0x7F == 0x7F and oq[8, 40] & 0x7F == 0x7F and oq[9, 5] == 0x7E and oq[9, 70] == 0xFE
    if dtype == "float32":  # (torch's conversion to bf16 does not keep a NaN's sign)
        assert oq[7, 3] == 0x7F and oq[8, 40] == 0xFF
    # and the inverse maps agree on everything finite
    back, oback = host.dequantize(q, sc).numpy(), mxfp8.mx_dequantize(oq, osc)
    fin = np.isfinite(oback)
    assert np.array_equal(back[fin], oback[fin]) and np.array_equal(np.isnan(back), np.isnan(oback))

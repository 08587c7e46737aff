"""Parity of the small kernels of a full decode step (embedding rows, the two RMSNorm forms, greedy arg-max) against the
CPU oracle, through the C ABI, on the GPU.

Bars: embedding rows and arg-max indices exact; the grouped norm within the reference test's bound (one BF16 ulp of
bf16(w * (x * r)), tests/test_mova_kernels.c:361-374); the Qwen norm within max-rel-err 1e-5 (tests/test_qwen4_kernels.c:61);
the arg-max probability within 1e-5 relative."""
import numpy as np
import pytest

from nanoseedlm_amd import packs
from test_gpu_kernels import NAMES, be, make_pack, slice_of   # noqa: F401  (be is a fixture)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fmt", [packs.MF_BF16, packs.MF_Q8, packs.MF_Q4, packs.MF_SEED4P4, packs.MF_SEED4])
def test_embed_rows_exact(be, oracle, fmt):
    rng = np.random.default_rng(300 + fmt)
    V, d = 40, 320
    p = make_pack(rng, fmt, 1, V, d)
    ids = np.array([7, 0, 39, 7], dtype=np.int32)
    got = be.kt_embed(p, ids)
    want = packs.bf16_bits_to_f32(oracle.slice_bf16(fmt, slice_of(oracle, p, 0), V, d))[ids]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), NAMES[fmt]


@pytest.mark.parametrize("d,T", [(256, 3), (2048, 5), (2880, 2), (16384, 1)])
def test_gnorm(be, oracle, d, T):
    rng = np.random.default_rng(d + T)
    x = packs.round_bf16((rng.standard_normal((T, d)) * 3).astype(np.float32))
    wb = packs.f32_to_bf16_bits((1 + 0.3 * rng.standard_normal(d)).astype(np.float32))
    got = be.kt_gnorm(x, wb, 1e-6)
    want = oracle.gnorm(x, wb, 1e-6)
    # both round the same product to BF16: equal, or one BF16 step apart where the f32 product sits on a rounding edge
    w = packs.bf16_bits_to_f32(wb).astype(np.float64)
    hw = d // 2
    xs = x.astype(np.float64).reshape(T, 2, hw)
    r = 1.0 / np.sqrt((xs ** 2).mean(-1, keepdims=True) + 1e-6)
    exact = (xs * r).reshape(T, d) * w
    assert np.all(np.abs(got - exact) <= np.abs(exact) * (2.0 ** -8 + 1e-6) + 1e-30)
    assert np.array_equal(got, packs.round_bf16(got))
    assert np.mean(got == want) > 0.995


@pytest.mark.parametrize("ln,g,T", [(2048, 2048, 3), (4096, 128, 2), (8192, 8192, 1), (768, 256, 4)])
def test_norm1p(be, oracle, ln, g, T):
    rng = np.random.default_rng(ln + g)
    x = rng.standard_normal((T, ln)).astype(np.float32)
    w = (0.2 * rng.standard_normal(ln)).astype(np.float32)
    got = be.kt_q4_norm1p(x, g, w, 1e-6)
    want = oracle.norm1p(x, g, w, 1e-6)
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) < 1e-5


def test_argmax_ties_and_probability(be, oracle):
    rng = np.random.default_rng(11)
    V = 250624   # the reference test's size (tests/test_mova_kernels.c:563)
    lg = packs.round_bf16((rng.standard_normal((2, V)) * 3).astype(np.float32))
    lg[0, 123456] = 50
    lg[0, 200000] = 50
    lg[1, 99] = 60
    assert be.kt_argmax(lg).tolist() == [123456, 99]
    out, prob = be.kt_argmax(lg, with_prob=True)
    oi, op = oracle.argmax(lg, with_prob=True)
    assert np.array_equal(out, oi)
    assert np.allclose(prob, op, rtol=1e-5)
    # ragged sizes (no 16-byte multiple), the vocabulary of the full model, a row without a finite maximum
    for V in (1, 7, 151936, 151937):
        l2 = rng.standard_normal((3, V)).astype(np.float32)
        assert np.array_equal(be.kt_argmax(l2), oracle.argmax(l2))
    assert be.kt_argmax(np.full((1, 33), -np.inf, dtype=np.float32)).tolist() == [0]

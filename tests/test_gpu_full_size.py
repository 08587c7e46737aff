"""The benchmark configurations at their full sizes, on the GPU.

Where the oracle finishes in seconds the whole result is compared (C0, and the C2 layer step on the experts the GPU chose);
for the 60-GFLOP prefill GEMM a random sample of weight rows is checked against the oracle over every token, and the whole
result through properties that do not depend on the size: linearity in the activations, invariance under a permutation of
the tokens, and zero activations giving zeros."""
import numpy as np
import pytest

from nanoseedlm_amd import packs
from test_gpu_kernels import F32B, be, close_bf, slice_of   # noqa: F401  (be is a fixture)

pytestmark = pytest.mark.gpu


def test_c0_dense_gemv_4096(be, oracle):
    rng = np.random.default_rng(4096)
    R = K = 4096
    p = packs.seed4p4(rng, 1, R, K, eb=-22)
    x = rng.standard_normal((1, K)).astype(np.float32)
    y = be.kt_mv(p, x)
    ref, mag = oracle.mv_double(p["fmt"], slice_of(oracle, p, 0), R, K, x[0])
    ref, mag = ref[0], mag[0]
    assert np.all(close_bf(y[0], ref, F32B * mag))
    be.kt().kt_store_f32(1)
    try:
        yf = be.kt_mv(p, x)
    finally:
        be.kt().kt_store_f32(0)
    assert np.max(np.abs(yf[0] - ref)) / np.max(np.abs(ref)) < 2e-3          # the fp32-accumulate bar (measured ~1e-6)


def test_c1_prefill_gemm_14336x4096x512(be, oracle):
    rng = np.random.default_rng(14336)
    R, K, T = 14336, 4096, 512
    p = packs.seed4p4(rng, 1, R, K, eb=-22)
    x = packs.round_bf16(rng.standard_normal((T, K)).astype(np.float32))
    y = be.kt_mm_plain(p, x, packed=1)
    # a sample of rows against the oracle: BF16-rounded weights, BF16 activations, f32 accumulate, BF16 store
    rows = np.sort(rng.choice(R, size=48, replace=False))
    w = oracle.rows_f32(p["fmt"], slice_of(oracle, p, 0), R, K)
    wb = packs.round_bf16(w[rows]).astype(np.float64)
    ref = x.astype(np.float64) @ wb.T
    mag = np.abs(x).astype(np.float64) @ np.abs(wb).T
    got = y[:, rows].astype(np.float64)
    assert np.all(np.abs(got - ref) <= np.abs(ref) / 128.0 + F32B * mag + 1e-30)
    assert np.max(np.abs(got - ref)) / np.max(np.abs(ref)) < 1e-2           # the BF16 MFMA bar
    # every output is a BF16 value (the store rounds)
    assert np.array_equal(y, packs.round_bf16(y))
    # permuting the tokens permutes the rows of Y, bit for bit (no token sees its neighbours)
    perm = rng.permutation(T)
    assert np.array_equal(be.kt_mm_plain(p, x[perm], packed=1), y[perm])
    # zero activations give zeros; linearity on activations with disjoint support (their sum is exact in BF16)
    x1, x2 = x.copy(), x.copy()
    x1[:, K // 2:] = 0
    x2[:, :K // 2] = 0
    assert not np.any(be.kt_mm_plain(p, np.zeros_like(x), packed=1))
    be.kt().kt_store_f32(1)
    try:
        yf = be.kt_mm_plain(p, x, packed=1).astype(np.float64)
        y12 = be.kt_mm_plain(p, x1, packed=1).astype(np.float64) + be.kt_mm_plain(p, x2, packed=1)
    finally:
        be.kt().kt_store_f32(0)
    scale = np.max(np.abs(yf))
    assert np.max(np.abs(yf - y12)) <= 1e-5 * scale                          # f32 accumulation order only


@pytest.mark.parametrize("T", [1, 8])
def test_c2_layer_step_128_experts(oracle, T):
    from nanoseedlm_amd import moe
    from test_gpu_moe import expert_ref
    rng = np.random.default_rng(128 + T)
    E, k, d, ff = 128, 8, 2048, 768
    st = moe.MoeStack(1, E, k, d, ff, fmt=packs.MF_SEED4P4, router=moe.ROUTE_SOFTMAX, max_rows=8)
    gate, up, down = (packs.seed4p4(rng, E, ff, d, eb=-22), packs.seed4p4(rng, E, ff, d, eb=-22), packs.seed4p4(rng, E, d, ff, eb=-22))
    rw = packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.02).astype(np.float32))
    st.set_layer(0, gate, up, down, rw)
    st.finalize()
    xn = packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))
    dx, dio = moe.DevBuf.from_array(xn), moe.DevBuf(4 * T * d)
    st.step(None, 0, dx.ptr, T, dio.ptr)
    ind, wt = st.last_routing(T)
    out = dio.to_array(np.float32, (T, d))
    assert st.fused_error() == 0
    # the routing against the oracle on BF16-rounded logits of its own (near-ties may move by a BF16 flip of a logit)
    W = packs.bf16_bits_to_f32(rw).astype(np.float64)
    lg = packs.round_bf16((xn.astype(np.float64) @ W.T).astype(np.float32))
    oi, _ = oracle.route_softmax(lg, k)
    assert np.mean([len(set(ind[t]) & set(oi[t])) / k for t in range(T)]) >= 0.9
    assert np.allclose(wt.sum(1), 1.0, atol=1e-5)
    # the layer output from the GPU's own routing, token 0 and the last token
    for t in sorted({0, T - 1}):
        ys = np.stack([expert_ref(oracle, gate, up, down, int(ind[t, j]), xn[t], gemm=False) for j in range(k)])
        want = (wt[t].astype(np.float64)[:, None] * ys).sum(0)
        tol = 2e-2 * np.abs(wt[t].astype(np.float64)[:, None] * ys).sum(0) + 1e-6
        assert np.all(np.abs(out[t] - want) <= tol)
    # the same step through the five separate launchers: the same bits
    st.set_fused(0)
    dio2 = moe.DevBuf(4 * T * d)
    st.step(None, 0, dx.ptr, T, dio2.ptr)
    assert np.array_equal(out.view(np.uint32), dio2.to_array(np.float32, (T, d)).view(np.uint32))
    st.close()

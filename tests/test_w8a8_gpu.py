"""GPU parity of the W8A8 path (per-row INT8 activation quantisation, int8 MFMA GEMM, scale /
zero / sum dequantisation) against the oracle's restatement of
MMHelper::onednn_amx_gemm_f32s8f32_compute (reference src/utils/matmul_helper.h:2762-2965)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def xh():
    from xfastertransformer_amd import capi
    capi.init(0)
    return capi


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


@pytest.mark.parametrize("M,K", [(1, 4096), (7, 512), (33, 11008), (5, 1008)])
def test_activation_quantisation_bit_exact(xh, orc, M, K):
    rng = np.random.default_rng(M + K)
    A = orc.round_bf16(rng.standard_normal((M, K)) * 2.0 + 0.3)
    ad = xh.DeviceBuffer.from_numpy(orc.to_bf16(A))
    qa, s, z, sm, ldq = xh.w8a8_quantize_rows(ad.ptr, xh.BF16, M, K, K)
    xh.synchronize()
    eq, es, ez, esm = orc.w8a8_quantize_rows(A)
    got_q = qa.to_numpy(np.int8, (M, ldq))[:, :K]
    assert np.array_equal(got_q, eq)
    assert np.array_equal(s.to_numpy(np.float32, M).view(np.uint32), es.view(np.uint32))
    assert np.array_equal(z.to_numpy(np.float32, M).view(np.uint32), ez.view(np.uint32))
    assert np.array_equal(sm.to_numpy(np.float32, M).view(np.uint32), esm.view(np.uint32))


@pytest.mark.parametrize("M", [1, 8, 17, 32, 70])
@pytest.mark.parametrize("K,N", [(4096, 4096), (512, 80), (11008, 256), (1008, 48)])
def test_w8a8_gemm_vs_oracle(xh, orc, M, K, N):
    if (K, N) == (4096, 4096) and M not in (1, 32):
        pytest.skip("large shape covered at M=1 and M=32")
    print(f"case M={M} K={K} N={N}", flush=True)
    rng = np.random.default_rng(M * 3 + N)
    W = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    w = orc.quantize(orc.W_W8A8, W)
    w.zero = (rng.standard_normal(N) * 0.002).astype(np.float32)  # exercise the sumA*zeroB term
    A = orc.round_bf16(rng.standard_normal((M, K)) + 0.2)
    dw = xh.Weight(xh.W_W8A8, K, N, w.q, w.scale, w.zero)
    assert np.array_equal(dw.unpack(), w.q)
    ad = xh.DeviceBuffer.from_numpy(orc.to_bf16(A))
    cd = xh.DeviceBuffer(M * N * 4)
    # one call: quantise + GEMM
    xh.gemm(dw, ad.ptr, M, K, cd.ptr, N, xh.F32)
    xh.synchronize()
    got = cd.to_numpy(np.float32, (M, N))
    exp = orc.qgemm(w, A)
    # integer accumulation is exact and the dequantisation is evaluated in the same order
    assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), np.abs(got - exp).max()
    # against the unquantised product the error is the quantisation noise of A and W
    assert np.abs(got - (A.astype(np.float64) @ W + A.astype(np.float64).sum(1, keepdims=True) * w.zero)).max() < 0.1 * np.sqrt(K / 4096.0) + 0.05
    # epilogue through the two-call form
    res = rng.standard_normal((M, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    qa, s, z, sm, ldq = xh.w8a8_quantize_rows(ad.ptr, xh.BF16, M, K, K)
    rd, bd = xh.DeviceBuffer.from_numpy(res), xh.DeviceBuffer.from_numpy(bias)
    xh.gemm_w8a8(dw, M, qa, ldq, s, z, sm, cd.ptr, N, xh.F32, xh.EPI_RESIDENTIAL, bd.ptr, rd.ptr, N)
    xh.synchronize()
    exp2 = orc.qgemm(w, A, orc.EPI_RESIDENTIAL, bias=bias, res=res)
    assert np.abs(cd.to_numpy(np.float32, (M, N)) - exp2).max() < 1e-5
    dw.free()


@pytest.mark.parametrize("M,K,N", [(256, 4096, 1024), (2048, 1024, 1024), (100, 1008, 176), (2011, 512, 4096)])
def test_w8a8_large_m_bit_exact(xh, orc, M, K, N):
    """More than 32 rows take the block-tiled int8 MFMA kernel: the same integers and the same
    dequantisation order as the M <= 32 kernel, so still bit-identical to the oracle."""
    print(f"case M={M} K={K} N={N}", flush=True)
    rng = np.random.default_rng(M + K + N)
    w = orc.quantize(orc.W_W8A8, (rng.standard_normal((K, N)) * 0.02).astype(np.float32))
    w.zero = (rng.standard_normal(N) * 0.002).astype(np.float32)
    A = orc.round_bf16(rng.standard_normal((M, K)) + 0.2)
    dw = xh.Weight(xh.W_W8A8, K, N, w.q, w.scale, w.zero)
    ad = xh.DeviceBuffer.from_numpy(orc.to_bf16(A))
    cd = xh.DeviceBuffer(M * N * 4)
    xh.gemm(dw, ad.ptr, M, K, cd.ptr, N, xh.F32)
    xh.synchronize()
    got = cd.to_numpy(np.float32, (M, N))
    exp = orc.qgemm(w, A)
    assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), np.abs(got - exp).max()
    res = rng.standard_normal((M, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    qa, s, z, sm, ldq = xh.w8a8_quantize_rows(ad.ptr, xh.BF16, M, K, K)
    rd, bd = xh.DeviceBuffer.from_numpy(res), xh.DeviceBuffer.from_numpy(bias)
    for epi in (xh.EPI_RESIDENTIAL, xh.EPI_BIAS, xh.EPI_SILU):
        xh.gemm_w8a8(dw, M, qa, ldq, s, z, sm, cd.ptr, N, xh.F32, epi, bd.ptr, rd.ptr, N)
        xh.synchronize()
        e2 = orc.qgemm(w, A, epi, bias=bias, res=res)
        assert np.abs(cd.to_numpy(np.float32, (M, N)) - e2).max() < 2e-4
    dw.free()


def test_w8a8_model_shape_rows_2048(xh, orc):
    """[2048, 4096] x [4096, 4096] at the model's size: sampled rows against the oracle (rows are
    independent in this path), every output finite."""
    M, K, N = 2048, 4096, 4096
    rng = np.random.default_rng(5)
    w = orc.quantize(orc.W_W8A8, (rng.standard_normal((K, N)) * 0.02).astype(np.float32))
    A = orc.round_bf16(rng.standard_normal((M, K)))
    dw = xh.Weight(xh.W_W8A8, K, N, w.q, w.scale, w.zero)
    ad = xh.DeviceBuffer.from_numpy(orc.to_bf16(A))
    cd = xh.DeviceBuffer(M * N * 4)
    xh.gemm(dw, ad.ptr, M, K, cd.ptr, N, xh.F32)
    xh.synchronize()
    got = cd.to_numpy(np.float32, (M, N))
    assert np.isfinite(got).all()
    rows = np.array([0, 1, 31, 32, 127, 128, 1000, 2046, 2047])
    exp = orc.qgemm(w, A[rows])
    assert np.array_equal(got[rows].view(np.uint32), exp.view(np.uint32))


def test_w8a8_many_tiles_bit_exact(xh, orc):
    """Enough 128 x 128 tiles for three workgroups on every CU (the tile taken then).  Ragged M and N, sampled rows
    against the oracle (rows are independent), plain and residual epilogues, bf16 output."""
    M, K, N = 3000, 512, 11024
    rng = np.random.default_rng(77)
    w = orc.quantize(orc.W_W8A8, (rng.standard_normal((K, N)) * 0.02).astype(np.float32))
    w.zero = (rng.standard_normal(N) * 0.002).astype(np.float32)
    A = orc.round_bf16(rng.standard_normal((M, K)) + 0.1)
    dw = xh.Weight(xh.W_W8A8, K, N, w.q, w.scale, w.zero)
    ad = xh.DeviceBuffer.from_numpy(orc.to_bf16(A))
    cd = xh.DeviceBuffer(M * N * 4)
    xh.gemm(dw, ad.ptr, M, K, cd.ptr, N, xh.F32)
    xh.synchronize()
    got = cd.to_numpy(np.float32, (M, N))
    assert np.isfinite(got).all()
    rows = np.array([0, 1, 31, 32, 127, 128, 129, 255, 256, 257, 383, 384, 511, 512, 1000, 1279, 1280, 2047, 2048, 2815, 2816, 2998, 2999])
    exp = orc.qgemm(w, A[rows])
    assert np.array_equal(got[rows].view(np.uint32), exp.view(np.uint32)), np.abs(got[rows] - exp).max()
    res = rng.standard_normal((M, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    qa, s, z, sm, ldq = xh.w8a8_quantize_rows(ad.ptr, xh.BF16, M, K, K)
    rd, bd = xh.DeviceBuffer.from_numpy(res), xh.DeviceBuffer.from_numpy(bias)
    xh.gemm_w8a8(dw, M, qa, ldq, s, z, sm, cd.ptr, N, xh.F32, xh.EPI_RESIDENTIAL, bd.ptr, rd.ptr, N)
    xh.synchronize()
    e2 = orc.qgemm(w, A[rows], orc.EPI_RESIDENTIAL, bias=bias, res=res[rows])
    assert np.abs(cd.to_numpy(np.float32, (M, N))[rows] - e2).max() < 2e-4
    c16 = xh.DeviceBuffer(M * N * 2)
    xh.gemm(dw, ad.ptr, M, K, c16.ptr, N, xh.BF16)
    xh.synchronize()
    got16 = c16.to_numpy(np.uint16, (M, N))
    assert np.array_equal(got16[rows], orc.to_bf16(exp))
    dw.free()

"""GPU parity of the weight-only GEMM at 17 .. 64 activation rows (batch-32 decode, expert GEMMs), the range
where the few-row kernel hands over to the tiled one: every epilogue, the SwiGLU pairing, ragged K and N, row
pitches wider than the matrices (NaN behind K, a fill pattern behind N), against the CPU oracle through the
C-ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

KINDS = {"int8": 0, "uint4": 1}


@pytest.fixture(scope="module")
def xh():
    from xfastertransformer_amd import capi
    capi.init(0)
    return capi


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


def _weights(orc, kind, K, N, seed, asym_int8=False):
    rng = np.random.default_rng(seed)
    W = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    w = orc.quantize(kind, W)
    if asym_int8:
        w.zero = (rng.standard_normal(N) * 0.01).astype(np.float32)
    return w


def _gemm(xh, orc, dw, A, M, K, N, c_dtype, epi=0, bias=None, res=None, gamma=1.0, lda=None, ldc=None):
    lda = lda or K
    ldc = ldc or N
    a_host = np.zeros((M, lda), np.uint16)
    a_host[:, :K] = orc.to_bf16(A)
    if lda > K:
        a_host[:, K:] = 0x7FC0  # NaN past K: must never be read into a sum
    a_dev = xh.DeviceBuffer.from_numpy(a_host)
    esz = 4 if c_dtype == xh.F32 else 2
    fill = np.full((M, ldc), 0x5A5A5A5A if esz == 4 else 0x5A5A, np.uint32 if esz == 4 else np.uint16)
    c_dev = xh.DeviceBuffer.from_numpy(fill)
    b_dev = None if bias is None else xh.DeviceBuffer.from_numpy(bias)
    r_dev = None if res is None else xh.DeviceBuffer.from_numpy(res)
    xh.gemm(dw, a_dev.ptr, M, lda, c_dev.ptr, ldc, c_dtype, epi, None if b_dev is None else b_dev.ptr,
            None if r_dev is None else r_dev.ptr, N, xh.F32, gamma)
    xh.synchronize()
    raw = c_dev.to_numpy(fill.dtype, (M, ldc))
    assert np.array_equal(raw[:, N:], fill[:, N:]), "wrote past N"
    if esz == 4:
        return raw[:, :N].view(np.float32)
    return xh.bf16_bits_to_f32(np.ascontiguousarray(raw[:, :N]))


@pytest.mark.parametrize("kind", ["int8", "uint4"])
@pytest.mark.parametrize("M", [17, 31, 32, 33, 48, 64])
@pytest.mark.parametrize("K,N", [(4096, 4096), (512, 80), (1000, 250), (11008, 512), (2048, 6144)])
def test_rows17_64_gemm_vs_oracle(xh, orc, kind, M, K, N):
    if (K, N) in ((4096, 4096), (2048, 6144)) and M not in (32, 64):
        pytest.skip("large shapes covered at M=32 and M=64")
    print(f"case kind={kind} M={M} K={K} N={N}", flush=True)
    k = KINDS[kind]
    w = _weights(orc, k, K, N, 300 + M, asym_int8=(kind == "int8" and N in (80, 250)))
    rng = np.random.default_rng(400 + M)
    A = orc.round_bf16(rng.standard_normal((M, K)))
    dw = xh.Weight(k, K, N, w.q, w.scale, w.zero)
    exp = orc.qgemm(w, A)
    got32 = _gemm(xh, orc, dw, A, M, K, N, xh.F32, lda=K + 8, ldc=N + 3)
    assert np.abs(got32 - exp).max() < 2e-3, np.abs(got32 - exp).max()
    got16 = _gemm(xh, orc, dw, A, M, K, N, xh.BF16, ldc=N + 5)
    assert (np.abs(got16 - exp) <= 2e-3 + np.abs(exp) * 2.0 ** -8).all()
    dw.free()


@pytest.mark.parametrize("kind", ["int8", "uint4"])
@pytest.mark.parametrize("epi", ["bias", "silu", "gelu", "resmul", "residential", "residential_bias", "resext"])
def test_rows17_64_gemm_epilogues(xh, orc, kind, epi):
    M, K, N = 40, 1024, 272
    w = _weights(orc, KINDS[kind], K, N, 320)
    rng = np.random.default_rng(321)
    A = orc.round_bf16(rng.standard_normal((M, K)))
    bias = rng.standard_normal(N).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    dw = xh.Weight(KINDS[kind], K, N, w.q, w.scale, w.zero)
    table = {"bias": (orc.EPI_BIAS, bias, None), "silu": (orc.EPI_SILU, None, None),
             "gelu": (orc.EPI_GELU, None, None), "resmul": (orc.EPI_RESMUL, None, res),
             "residential": (orc.EPI_RESIDENTIAL, None, res), "residential_bias": (orc.EPI_RESIDENTIAL, bias, res),
             "resext": (orc.EPI_RESEXT, None, res)}
    e, b, r = table[epi]
    exp = orc.qgemm(w, A, e, bias=b, res=r, gamma=0.5)
    got = _gemm(xh, orc, dw, A, M, K, N, xh.F32, e, b, r, 0.5)
    assert np.abs(got - exp).max() < 2e-3
    dw.free()


@pytest.mark.parametrize("kind", ["int8", "uint4"])
@pytest.mark.parametrize("M,K,I", [(24, 1024, 2816), (64, 4096, 11008), (32, 2048, 1408)])
def test_rows17_64_gateup_silu_vs_oracle(xh, orc, kind, M, K, I):
    print(f"case kind={kind} M={M} K={K} I={I}", flush=True)
    k = KINDS[kind]
    w = _weights(orc, k, K, 2 * I, 330)
    rng = np.random.default_rng(331 + M)
    A = orc.round_bf16(rng.standard_normal((M, K)))
    dw = xh.Weight(k, K, 2 * I, w.q, w.scale, w.zero, flags=xh.WF_GATEUP)
    a_dev = xh.DeviceBuffer.from_numpy(orc.to_bf16(A))
    o_dev = xh.DeviceBuffer(M * I * 4)
    xh.gemm_gateup_silu(dw, a_dev.ptr, M, K, o_dev.ptr, I, xh.F32)
    xh.synchronize()
    got = o_dev.to_numpy(np.float32, (M, I))
    exp = orc.silu_sum(orc.qgemm(w, A))
    assert np.abs(got - exp).max() < 2e-3 + 2e-4 * np.abs(exp).max()
    dw.free()


@pytest.mark.parametrize("kind", ["int8", "int8_asym", "uint4", "nf4"])
@pytest.mark.parametrize("M,K,N", [(32, 1024, 12288), (20, 1024, 16400), (17, 576, 13000)])
def test_rows17_32_wide_column_blocks(xh, orc, kind, M, K, N):
    """At 17 .. 32 rows and more than two column tiles a CU, a workgroup takes 3 or 4 column tiles (one round over
    the CUs): the 768 tiles of a 7B QKV projection, a ragged tile count whose last block is mostly past N, a
    ragged K."""
    print(f"case kind={kind} M={M} K={K} N={N}", flush=True)
    k = {"int8": 0, "int8_asym": 0, "uint4": 1, "nf4": 2}[kind]
    w = _weights(orc, k, K, N, 350 + M, asym_int8=(kind == "int8_asym"))
    rng = np.random.default_rng(351 + M)
    A = orc.round_bf16(rng.standard_normal((M, K)))
    dw = xh.Weight(k, K, N, w.q, w.scale, w.zero)
    exp = orc.qgemm(w, A)
    got32 = _gemm(xh, orc, dw, A, M, K, N, xh.F32, lda=K + 8, ldc=N + 3)
    assert np.abs(got32 - exp).max() < 2e-3, np.abs(got32 - exp).max()
    res = rng.standard_normal((M, N)).astype(np.float32)
    exp_r = orc.qgemm(w, A, orc.EPI_RESIDENTIAL, res=res)
    got_r = _gemm(xh, orc, dw, A, M, K, N, xh.F32, orc.EPI_RESIDENTIAL, None, res)
    assert np.abs(got_r - exp_r).max() < 2e-3
    dw.free()


@pytest.mark.parametrize("kind", ["int8", "uint4", "nf4"])
@pytest.mark.parametrize("M,K,I", [(32, 1024, 11008), (24, 1024, 6000), (18, 512, 4112)])
def test_rows17_32_gateup_wide_column_blocks(xh, orc, kind, M, K, I):
    """SwiGLU pairs at 17 .. 32 rows with 6 (1376 tiles, the 7B gate/up) and 4 column tiles a workgroup."""
    print(f"case kind={kind} M={M} K={K} I={I}", flush=True)
    k = {"int8": 0, "uint4": 1, "nf4": 2}[kind]
    w = _weights(orc, k, K, 2 * I, 360)
    rng = np.random.default_rng(361 + M)
    A = orc.round_bf16(rng.standard_normal((M, K)))
    dw = xh.Weight(k, K, 2 * I, w.q, w.scale, w.zero, flags=xh.WF_GATEUP)
    a_dev = xh.DeviceBuffer.from_numpy(orc.to_bf16(A))
    o_dev = xh.DeviceBuffer(M * I * 4)
    xh.gemm_gateup_silu(dw, a_dev.ptr, M, K, o_dev.ptr, I, xh.F32)
    xh.synchronize()
    got = o_dev.to_numpy(np.float32, (M, I))
    exp = orc.silu_sum(orc.qgemm(w, A))
    assert np.abs(got - exp).max() < 2e-3 + 2e-4 * np.abs(exp).max()
    dw.free()


def test_rows17_64_bf16_weights_and_repeatability(xh, orc):
    """BF16 weights at 17 .. 64 rows; the summation order is fixed, so two runs agree to the bit."""
    rng = np.random.default_rng(340)
    K, N = 2048, 1000
    W = orc.round_bf16(rng.standard_normal((K, N)) * 0.05)
    dw = xh.Weight(xh.W_BF16, K, N, orc.to_bf16(W))
    for M in (20, 64):
        A = orc.round_bf16(rng.standard_normal((M, K)))
        got = _gemm(xh, orc, dw, A, M, K, N, xh.F32)
        assert np.abs(got - orc.gemm_f32(A, W)).max() < 2e-3
        again = _gemm(xh, orc, dw, A, M, K, N, xh.F32)
        assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    dw.free()

"""GPU parity: the decode chain's skinny matrix-core GEMM (and the weight transpose that feeds it) against a
float64 matmul of the same 16-bit operands, through the C ABI."""
import numpy as np
import pytest
import torch

import orc
from gpu_util import DEV, assert_close, dev, host, quant

pytestmark = pytest.mark.gpu

ops = pytest.importorskip("mamba_rs_amd.ops")

# (M, N, K): the 130m decode projections at batch 64 and 1, ragged M / N, the smallest K
SHAPES = [(64, 3072, 768), (64, 80, 1536), (64, 768, 1536), (1, 3072, 768), (1, 80, 1536), (5, 33, 32), (17, 100, 96),
          (48, 16, 2560), (33, 1000, 64), (64, 50, 1024), (128, 768, 1536), (97, 80, 1536), (100, 3072, 768),
          # one to four rows: lanes-along-the-row route (64 lanes per weight row at K % 512 == 0, 32 at K % 256 == 0)
          (1, 10240, 2560), (1, 192, 5120), (2, 2560, 5120), (3, 100, 512), (4, 33, 768), (1, 7, 256), (4, 3072, 768), (2, 50, 1280)]


@pytest.mark.parametrize("dtype", [orc.BF16, orc.F16])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("out_f32", [False, True])
def test_gemm_skinny_matches_f64_matmul(shape, dtype, out_f32):
    M, N, K = shape
    rng = np.random.default_rng(hash((shape, dtype)) & 0xFFFF)
    a = quant(rng.standard_normal((M, K)).astype(np.float32), dtype)
    w = quant((rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32), dtype)   # the reference's [K, N] layout
    print(f"case gemm_skinny shape={shape} dtype={dtype} out_f32={out_f32}", flush=True)
    wt = ops.transpose(dev(w, dtype))
    assert np.array_equal(host(wt), w.T)
    c = ops.gemm_skinny(dev(a, dtype), wt, out_f32=out_f32)
    ref = a.astype(np.float64) @ w.astype(np.float64)
    # f32 accumulation of exact 16-bit products: 1e-4 of the row scale when the result stays f32
    assert_close(host(c), ref, orc.F32 if out_f32 else dtype, "C")


# (M, N, K): the 2.8b decode projections at one to four 16-row tiles (whole and partly filled), N not a multiple of 16, a K
# shorter than the eight waves' ranges, a K that does not divide by them
# (small weights go to the 16 x 16 tiles reading the same tiled weight: the 130m decode projections, up to 128 rows)
TILED_SHAPES = [(16, 4096, 2080), (16, 10240, 2560), (64, 10240, 2560), (5, 2560, 5120), (23, 2560, 5120), (40, 2560, 5120), (64, 2560, 5120),
                (16, 200, 96), (33, 16, 32), (48, 1000, 1056), (1, 50, 256), (64, 8200, 64),
                (64, 3072, 768), (128, 768, 1536), (97, 80, 1536), (3, 3072, 768)]


@pytest.mark.parametrize("dtype", [orc.BF16, orc.F16])
@pytest.mark.parametrize("shape", TILED_SHAPES)
def test_gemm_tiled_matches_f64_matmul(shape, dtype):
    """The wide-model decode GEMM on a tiled weight (16 columns x 32 k of a matrix-core operand stored as one kilobyte):
    the tiling of the transposed weight, then the product against a float64 matmul, storage-type and f32 results."""
    M, N, K = shape
    rng = np.random.default_rng(hash((shape, dtype)) & 0xFFFF)
    a = quant(rng.standard_normal((M, K)).astype(np.float32), dtype)
    w = quant((rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32), dtype)
    print(f"case gemm_tiled shape={shape} dtype={dtype}", flush=True)
    wt = ops.transpose(dev(w, dtype))
    wp, n = ops.tile_weight(wt)
    assert n == N
    # tile (column tile t, k-step s) holds, for lane l, the 8 elements Wt[16 t + l % 16][32 s + 8 (l / 16) .. +7]
    tiles = host(wp.view(torch.int16)).reshape((N + 15) // 16, K // 32, 64, 8)
    wt_bits = host(wt.view(torch.int16))
    for t, s_, l in ((0, 0, 0), ((N - 1) // 16, K // 32 - 1, 37), ((N + 15) // 32, (K // 32) // 2, 63)):
        col = 16 * t + l % 16
        want = wt_bits[col, 32 * s_ + 8 * (l // 16): 32 * s_ + 8 * (l // 16) + 8] if col < N else np.zeros(8, np.int16)
        assert np.array_equal(tiles[t, s_, l], want), (t, s_, l)
    ref = a.astype(np.float64) @ w.astype(np.float64)
    for out_f32 in (False, True):
        c = ops.gemm_tiled(dev(a, dtype), wp, N, out_f32=out_f32)
        assert_close(host(c), ref, orc.F32 if out_f32 else dtype, "C")
    # strided rows of A
    big = dev(np.concatenate([a, a], axis=1), dtype)
    c = ops.gemm_tiled(big[:, K:], wp, N, out_f32=True)
    assert_close(host(c), ref, orc.F32, "C from strided rows")


def test_gemm_tiled_rejects_bad_arguments():
    wt = torch.zeros(32, 64, device=DEV, dtype=torch.bfloat16)
    wp, n = ops.tile_weight(wt)
    with pytest.raises(RuntimeError, match="skinny gemm"):
        ops.gemm_tiled(torch.zeros(129, 64, device=DEV, dtype=torch.bfloat16), wp, n)      # more than 128 rows
    with pytest.raises(ValueError):
        ops.tile_weight(torch.zeros(32, 48, device=DEV, dtype=torch.bfloat16))              # K % 32 != 0


@pytest.mark.parametrize("shape", [(1, 300, 256), (1, 3072, 768), (2, 40, 512), (3, 33, 128), (4, 1536, 1536), (4, 7, 384)])
def test_gemm_skinny_f32_storage_on_the_row_wise_route(shape):
    """f32 operands: one to four rows, lanes along the weight row, plain multiply-adds (K a multiple of 128)."""
    M, N, K = shape
    rng = np.random.default_rng(M * 1000 + N)
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    print(f"case gemm_skinny f32 shape={shape}", flush=True)
    wt = ops.transpose(dev(w))
    c = ops.gemm_skinny(dev(a), wt)
    assert_close(host(c), a.astype(np.float64) @ w.astype(np.float64), orc.F32, "C")
    from mamba_rs_amd import MambaHipError
    with pytest.raises(MambaHipError):   # five rows: f32 has no matrix-core route
        ops.gemm_skinny(dev(rng.standard_normal((5, K)).astype(np.float32)), wt)


def test_gemm_skinny_strided_rows_and_f32_transpose():
    """A may be a view into wider rows (e.g. a slice of a projection); transpose also serves f32 tables."""
    rng = np.random.default_rng(3)
    M, N, K = 12, 40, 64
    wide = quant(rng.standard_normal((M, 3 * K)).astype(np.float32), orc.BF16)
    w = quant(rng.standard_normal((K, N)).astype(np.float32), orc.BF16)
    a = dev(wide, orc.BF16)[:, K:2 * K]
    c = ops.gemm_skinny(a, ops.transpose(dev(w, orc.BF16)), out_f32=True)
    assert_close(host(c), wide[:, K:2 * K].astype(np.float64) @ w.astype(np.float64), orc.F32, "C (strided A)")
    f = rng.standard_normal((37, 53)).astype(np.float32)
    assert np.array_equal(host(ops.transpose(dev(f))), f.T)


def test_gemm_skinny_rejects_bad_arguments():
    from mamba_rs_amd import MambaHipError
    a = torch.zeros(129, 64, device=DEV, dtype=torch.bfloat16)
    wt = torch.zeros(16, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(MambaHipError) as e:   # M > 128
        ops.gemm_skinny(a, wt)
    assert e.value.code == -2
    with pytest.raises(MambaHipError) as e:   # K not a multiple of 32
        ops.gemm_skinny(torch.zeros(4, 48, device=DEV, dtype=torch.bfloat16), torch.zeros(16, 48, device=DEV, dtype=torch.bfloat16))
    assert e.value.code == -2
    with pytest.raises(MambaHipError) as e:   # f32 storage goes to the library GEMM, not here
        ops.gemm_skinny(torch.zeros(4, 64, device=DEV), torch.zeros(16, 64, device=DEV))
    assert e.value.code == -2

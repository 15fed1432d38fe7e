"""Matrix multiply on the device against the CPU checker.

Bars: bit-exact for integer types; fp32 within 1e-5 relative plus an absolute
term K*eps*max|a|*max|b| for summation order; fp16/bf16 (fp32 accumulation on
both sides) within rel 2e-3 / abs 1e-3.
"""
import numpy as np
import pytest

import golden_cases
import support
import tannic_amd as ta
from tannic_amd import ops

pytestmark = pytest.mark.gpu
SEED = 13
GEMM_GOLDEN = [c for c in golden_cases.TENSOR_CASES if c["op"] == "matmul"]

LAYOUTS = {
    "nn": ((5, 7), (7, 3), [], []),
    "nt": ((5, 7), (3, 7), [], [("transpose", (-1, -2))]),
    "tn": ((7, 5), (7, 3), [("transpose", (-1, -2))], []),
    "tt": ((7, 5), (3, 7), [("transpose", (-1, -2))], [("transpose", (-1, -2))]),
    "nn_mid": ((130, 70), (70, 190), [], []),
    "nt_mid": ((130, 72), (190, 72), [], [("transpose", (-1, -2))]),
    "tn_mid": ((72, 130), (72, 190), [("transpose", (-1, -2))], []),
    "tt_mid": ((72, 130), (190, 72), [("transpose", (-1, -2))], [("transpose", (-1, -2))]),
    "nt_tiles": ((256, 128), (384, 128), [], [("transpose", (-1, -2))]),
    "nn_tiles": ((256, 128), (128, 384), [], []),
    "batched": ((2, 3, 33, 40), (2, 3, 40, 17), [], []),
    "batch_broadcast": ((2, 1, 33, 40), (1, 3, 40, 17), [], []),
    "rank4_rank2_nt": ((2, 3, 20, 64), (48, 64), [], [("transpose", (-1, -2))]),
    "attention_scores": ((1, 4, 64, 32), (1, 4, 64, 32), [], [("transpose", (-1, -2))]),
    "attention_values": ((1, 4, 64, 64), (1, 4, 64, 32), [], []),
    "head_split_view": ((1, 64, 4, 32), (1, 64, 4, 32), [("transpose", (1, 2))], [("transpose", (1, 2)), ("transpose", (-1, -2))]),
    "single_row": ((1, 256), (96, 256), [], [("transpose", (-1, -2))]),
    "sixteen_rows": ((16, 256), (96, 256), [], [("transpose", (-1, -2))]),
    "single_column": ((64, 96), (1, 96), [], [("transpose", (-1, -2))]),
    "k_one": ((9, 1), (1, 11), [], []),
    # a matrix times a column (run as one row times the transposed matrix): plain, the matrix stored transposed, batches
    "matrix_vector": ((300, 512), (512, 1), [], []),
    "matrix_vector_transposed_matrix": ((512, 300), (512, 1), [("transpose", (-1, -2))], []),
    "matrix_vector_batched": ((3, 70, 256), (3, 256, 1), [], []),
    # many rows times a few columns (run transposed through the streaming kernel and turned back)
    "few_columns": ((600, 4096), (10, 4096), [], [("transpose", (-1, -2))]),
    "two_columns_of_a_wider_result": ((700, 4096), (32, 4096), [], [("index", (slice(3, 5), slice(None))), ("transpose", (-1, -2))]),
    # few rows: ragged K steps and columns, two row blocks, batches; a long K shared between blocks
    "skinny_17_rows_ragged": ((17, 72), (40, 72), [], [("transpose", (-1, -2))]),
    "skinny_batched": ((3, 5, 64), (3, 24, 64), [], [("transpose", (-1, -2))]),
    # few rows with whole 64-wide K windows (operands streamed through LDS): one and two row blocks, ragged columns, one
    # and two column blocks per wavefront, fewer windows than wavefronts, batches, rows longer than K (a view)
    "stream_1_row": ((1, 1024), (200, 1024), [], [("transpose", (-1, -2))]),
    "stream_16_rows_ragged_columns": ((16, 640), (90, 640), [], [("transpose", (-1, -2))]),
    "stream_20_rows_one_window": ((20, 64), (48, 64), [], [("transpose", (-1, -2))]),
    "stream_32_rows_many_columns": ((32, 128), (12840, 128), [], [("transpose", (-1, -2))]),
    "stream_5_rows_many_columns": ((5, 192), (12816, 192), [], [("transpose", (-1, -2))]),
    # 33 .. 64 rows over a small W (one product, K >= 256): three and four row blocks per wavefront; batches of such
    # products and shorter K stay on tiles
    "stream_40_rows": ((40, 320), (100, 320), [], [("transpose", (-1, -2))]),
    "stream_64_rows_ragged_columns": ((64, 256), (90, 256), [], [("transpose", (-1, -2))]),
    "stream_33_rows": ((33, 256), (50, 256), [], [("transpose", (-1, -2))]),
    "tiles_33_rows_batched": ((2, 33, 128), (2, 50, 128), [], [("transpose", (-1, -2))]),
    "tiles_64_rows_many_small_batches": ((40, 64, 64), (40, 64, 64), [], [("transpose", (-1, -2))]),
    "stream_49_rows_long_k": ((49, 2048), (24, 2048), [], [("transpose", (-1, -2))]),
    "stream_batched_views": ((3, 9, 320), (3, 70, 320), [("index", (Ellipsis, slice(0, 256)))], [("index", (Ellipsis, slice(64, 320))), ("transpose", (-1, -2))]),
    "split_k_nt": ((128, 1096), (136, 1096), [], [("transpose", (-1, -2))]),
    "split_k_nn": ((72, 2048), (2048, 64), [], []),
    # operands contiguous along M / N with ragged tiles and a K tail, in every tile size (the largest needs 200 tiles)
    "tn_tiles_ragged": ((200, 520), (200, 264), [("transpose", (-1, -2))], []),
    "tt_tiles_ragged": ((136, 264), (520, 136), [("transpose", (-1, -2))], [("transpose", (-1, -2))]),
    "tn_large_tiles_batched": ((50, 24, 264), (50, 24, 264), [("transpose", (-1, -2))], []),
    "nn_large_tiles_batched": ((50, 264, 72), (50, 72, 264), [], []),
    # K-contiguous operands that 16-byte loads cannot take: odd K, odd row pitch, a view starting at an odd column
    "nt_odd_k": ((130, 75), (190, 75), [], [("transpose", (-1, -2))]),
    "nt_odd_pitch_and_start": ((130, 77), (190, 79), [("index", (slice(None), slice(1, 73)))], [("index", (slice(None), slice(3, 75))), ("transpose", (-1, -2))]),
    "nt_odd_k_few_rows_batched": ((3, 40, 203), (3, 150, 203), [], [("transpose", (-1, -2))]),
    # the same for operands contiguous along M / N: odd extents, odd pitches, views that start at odd columns, fewer rows than
    # a 16-byte piece holds, odd batch strides, and tiles on every side of a 128 x 128 grid
    "nn_odd_extents": ((131, 75), (75, 197), [], []),
    "nn_odd_pitch_and_start": ((131, 75), (75, 203), [], [("index", (slice(None), slice(3, 200)))]),
    "tn_odd_pitch_and_start": ((77, 141), (77, 203), [("index", (slice(None), slice(1, 132))), ("transpose", (-1, -2))], [("index", (slice(None), slice(3, 200)))]),
    "tt_odd_extents": ((75, 131), (197, 75), [("transpose", (-1, -2))], [("transpose", (-1, -2))]),
    "tn_three_rows": ((200, 3), (200, 5), [("transpose", (-1, -2))], []),
    "nn_odd_batched": ((3, 41, 203), (3, 203, 151), [], []),
    "tn_odd_tiles": ((70, 259), (70, 385), [("transpose", (-1, -2))], []),
    # both operands K-contiguous, whole K steps, 200 large tiles: the tiles filled by direct global -> LDS loads
    # (rows past the end of both operands; one, two and three K steps)
    "nt_direct_one_step": ((50, 264, 64), (50, 264, 64), [], [("transpose", (-1, -2))]),
    "nt_direct_two_steps": ((50, 264, 128), (50, 264, 128), [], [("transpose", (-1, -2))]),
    "nt_direct_ragged_rows": ((10, 1000, 192), (10, 1096, 192), [], [("transpose", (-1, -2))]),
    # enough tiles of 128 x 128 to fill the chip (float64: wavefronts of 4 x 4 MFMA tiles, each walking all of K), a
    # thousand square (float64: 64 x 64 per workgroup, its wavefronts sharing K; under a K of 100 side by side), every layout
    "many_tiles_nt": ((2001, 40), (2039, 40), [], [("transpose", (-1, -2))]),
    "many_tiles_nn": ((2001, 40), (40, 2039), [], []),
    "many_tiles_tn": ((40, 2001), (40, 2039), [("transpose", (-1, -2))], []),
    "many_tiles_tt": ((40, 2001), (2039, 40), [("transpose", (-1, -2))], [("transpose", (-1, -2))]),
    "thousand_square_nt": ((1000, 200), (1010, 200), [], [("transpose", (-1, -2))]),
    "thousand_square_nn": ((1000, 200), (200, 1010), [], []),
    "thousand_square_tn": ((200, 1000), (200, 1010), [("transpose", (-1, -2))], []),
    "thousand_square_tt": ((200, 1000), (1010, 200), [("transpose", (-1, -2))], [("transpose", (-1, -2))]),
    "thousand_square_short_k_nt": ((1000, 100), (1010, 100), [], [("transpose", (-1, -2))]),
    "thousand_square_short_k_nn": ((1000, 100), (100, 1010), [], []),
    # at most eight rows times a matrix lying row by row (fp32: W read once along its rows, K shared between workgroups):
    # one row, a K no eight divides under columns that end inside a wavefront, x transposed, W a slice of a wider matrix
    "rows_nn_1_row": ((1, 1024), (1024, 512), [], []),
    "rows_nn_5_rows_ragged": ((5, 1003), (1003, 520), [], []),
    "rows_nn_8_rows_x_transposed": ((700, 8), (700, 1024), [("transpose", (-1, -2))], []),
    "rows_nn_3_rows_slice_of_w": ((3, 512), (512, 1100), [], [("index", (slice(None), slice(4, 1028)))]),
    "rows_nn_2_rows_long_k": ((2, 20000), (20000, 256), [], []),
    # few results under a long K (a workgroup per 4 x 4 results, its lanes striding over K): every layout, odd extents, batches
    "few_results_nt": ((48, 2047), (13, 2047), [], [("transpose", (-1, -2))]),
    "few_results_nn": ((20, 1500), (1500, 9), [], []),
    "few_results_tn": ((3000, 6), (3000, 8), [("transpose", (-1, -2))], []),
    "few_results_tt": ((1024, 33), (50, 1024), [("transpose", (-1, -2))], [("transpose", (-1, -2))]),
    "few_results_batched": ((5, 6, 1100), (5, 1100, 10), [], []),
    "rank4_rank2_nt_large": ((2, 3, 200, 320), (480, 320), [], [("transpose", (-1, -2))]),
    "stream_49_rows_long_k_wide": ((49, 2048), (400, 2048), [], [("transpose", (-1, -2))]),
}


@pytest.mark.parametrize("case", GEMM_GOLDEN, ids=lambda c: c["name"])
def test_reference_vectors_on_device(device, case):
    got = golden_cases.run(case, device)
    support.assert_close(got, golden_cases.expected_of(case), 1e-5, 1e-8, case["name"])


def operands(pair, layout, device, low=-1, high=1):
    sa, sb, va, vb = LAYOUTS[layout]
    ha, da = support.both(support.values_for(pair[0], SEED, 1, sa, low, high), pair[0], device)
    hb, db = support.both(support.values_for(pair[1], SEED, 2, sb, low, high), pair[1], device)
    k = support.apply_view(ha, va).shape[-1]
    return (support.apply_view(ha, va), support.apply_view(hb, vb)), (support.apply_view(da, va), support.apply_view(db, vb)), k


@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("dtype", [ta.float32, ta.float64], ids=str)
def test_float_gemm(device, dtype, layout):
    host, dev, k = operands((dtype, dtype), layout, device)
    want, got = ops.matmul(*host), ops.matmul(*dev)
    assert got.shape == want.shape and got.dtype is want.dtype
    eps = 2.0 ** -24 if dtype is ta.float32 else 2.0 ** -53
    support.assert_close(got.numpy(), want.numpy(), 1e-5 if dtype is ta.float32 else 1e-13, k * eps, f"gemm {dtype} {layout}")


@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_16bit_gemm_fp32_accumulate(device, dtype, layout):
    host, dev, k = operands((dtype, dtype), layout, device)
    want, got = ops.matmul(*host), ops.matmul(*dev)
    assert got.shape == want.shape and got.dtype is dtype
    rtol = 2e-3 if dtype is ta.float16 else 2.0 ** -7   # bf16 keeps 8 significant bits: one ulp is 2^-7 relative
    support.assert_close(got.numpy(), want.numpy(), rtol, 1e-3, f"gemm {dtype} {layout}")


@pytest.mark.parametrize("layout", ["nn", "nt_mid", "tn_mid", "batched", "batch_broadcast", "rank4_rank2_nt",
                                    "single_row", "sixteen_rows", "stream_16_rows_ragged_columns", "stream_batched_views", "matrix_vector",
                                    "matrix_vector_batched", "few_results_nt", "few_results_nn", "few_results_tt", "few_results_batched"])
@pytest.mark.parametrize("pair", [(ta.int8, ta.int8), (ta.int16, ta.int32), (ta.int32, ta.int32), (ta.int64, ta.int8)], ids=lambda p: f"{p[0]}-{p[1]}")
def test_integer_gemm_bit_exact(device, pair, layout):
    host, dev, _ = operands(pair, layout, device, -100, 100)
    want, got = ops.matmul(*host), ops.matmul(*dev)
    assert got.dtype is want.dtype
    support.assert_bit_exact(got.storage(), want.storage(), f"gemm {pair} {layout}")


@pytest.mark.parametrize("shape", [((300, 256), (520, 256)), ((16, 300, 128), (16, 520, 128)), ((50, 264, 128), (50, 264, 128)), ((2, 3, 70, 384), (136, 384)),
                                   ((4096, 512), (1024, 512)), ((1, 512), (1024, 512)), ((16, 256), (130, 256)), ((3, 5, 128), (3, 70, 128)),
                                   ((130, 384), (1001, 384)), ((70, 200), (333, 200)), ((300, 1000), (77, 1000)),
                                   # at most 32 rows over whole windows of 128 k: streamed (one and two row blocks, one and two column
                                   # blocks per wavefront, ragged columns, a K the four wavefronts do not share evenly, batches)
                                   ((32, 128), (12840, 128)), ((17, 1280), (200, 1280)), ((5, 640), (12816, 640)), ((4, 9, 384), (4, 90, 384)),
                                   ((2, 3, 20, 256), (48, 256))],
                         ids=lambda s: "x".join(map(str, s[0])) + "." + "x".join(map(str, s[1])) + "T")
def test_int8_gemm_on_matrix_cores_is_bit_exact(device, shape):
    """int8 x int8 -> int32 with both operands K-contiguous and K a multiple of 128: the tiled kernels on
    v_mfma_i32_16x16x64_i8 in each tile size (128 x 128, 256 x 128, 256 x 256; ragged rows and columns, batches, a
    broadcast second operand; few rows, which stream W once; a number of columns no quad divides; K that is
    not a multiple of 128, which goes through zero-padded copies of both operands).  Integer sums are exact, so the checker's sequential loop and numpy agree bit for bit."""
    sa, sb = shape
    a = support.integers(SEED, 31, sa, -128, 128).astype(np.int8)
    b = support.integers(SEED, 32, sb, -128, 128).astype(np.int8)
    (ha, da), (hb, db) = support.both(a, ta.int8, device), support.both(b, ta.int8, device)
    got = ops.matmul(da, db.transpose())
    assert got.dtype is ta.int32
    want = np.matmul(a.astype(np.int64), np.swapaxes(b.astype(np.int64), -1, -2)).astype(np.int32)
    support.assert_bit_exact(got.storage(), want, f"int8 gemm {sa} x {sb}^T against numpy")
    if int(np.prod(sa)) * sb[-2] < 40_000_000:
        support.assert_bit_exact(got.storage(), ops.matmul(ha, hb.transpose()).storage(), f"int8 gemm {sa} x {sb}^T against the checker")


@pytest.mark.parametrize("shape", [((6, 64, 300), (6, 337, 300), "nt"), ((5, 70, 260), (5, 260, 129), "nn"), ((4, 200, 64), (4, 49, 200), "tt"),
                                   ((3, 40, 384), (1, 384, 72), "nn"), ((1, 33, 130), (7, 90, 130), "nt")], ids=lambda s: s[2] + "-" + "x".join(map(str, s[0])))
def test_int8_batches_in_other_layouts_are_bit_exact(device, shape):
    """A batch of int8 products along one dim whose operands are not K-contiguous, or whose K no 128 divides: every
    product's operands are copied into K-contiguous zero-padded rows (an operand all products share, once) and the batch
    runs on the matrix cores; bit for bit equal to numpy's int64 product."""
    sa, sb, layout = shape
    a = support.integers(SEED, 41, sa, -128, 128).astype(np.int8)
    b = support.integers(SEED, 42, sb, -128, 128).astype(np.int8)
    (ha, da), (hb, db) = support.both(a, ta.int8, device), support.both(b, ta.int8, device)
    va, vb = (da.transpose() if layout[0] == "t" else da), (db.transpose() if layout[1] == "t" else db)
    na, nb = (np.swapaxes(a, -1, -2) if layout[0] == "t" else a), (np.swapaxes(b, -1, -2) if layout[1] == "t" else b)
    got = ops.matmul(va, vb)
    want = np.matmul(na.astype(np.int64), nb.astype(np.int64)).astype(np.int32)
    assert got.dtype is ta.int32 and got.shape == want.shape
    support.assert_bit_exact(got.storage(), want, f"int8 batch {sa} x {sb} {layout}")


@pytest.mark.parametrize("layout", ["nn", "tn", "tt"])
def test_int8_gemm_in_other_layouts_is_bit_exact(device, layout):
    """int8 operands that are not contiguous along K (and a K of 300) are copied into K-contiguous rows, zero-padded to
    whole steps, and multiplied on the matrix cores."""
    m, n, k = 200, 170, 300
    a = support.integers(SEED, 33, (k, m) if layout[0] == "t" else (m, k), -128, 128).astype(np.int8)
    b = support.integers(SEED, 34, (n, k) if layout[1] == "t" else (k, n), -128, 128).astype(np.int8)
    (ha, da), (hb, db) = support.both(a, ta.int8, device), support.both(b, ta.int8, device)
    view = lambda t, transposed: t.transpose() if transposed else t
    got = ops.matmul(view(da, layout[0] == "t"), view(db, layout[1] == "t"))
    want = ops.matmul(view(ha, layout[0] == "t"), view(hb, layout[1] == "t"))
    assert got.dtype is ta.int32 and got.shape == (m, n)
    support.assert_bit_exact(got.storage(), want.storage(), f"int8 gemm {layout}")


REPACKED = {
    # large enough to be worth a copy: a second operand whose rows start at odd addresses, an odd K (zeros added to both), a
    # first operand stored transposed with an odd number of rows, and a single row of a transposed first operand
    "nn_odd_columns": ((300, 1032), (1032, 1001), [], []),
    "nn_odd_k": ((260, 1001), (1001, 1040), [], []),
    "tn_odd_rows": ((1032, 301), (1032, 1000), [("transpose", (-1, -2))], []),
    "nt_odd_k_few_rows": ((8, 2049), (1500, 2049), [], [("transpose", (-1, -2))]),
    "tn_single_row": ((4096, 1), (4096, 520), [("transpose", (-1, -2))], []),
}


@pytest.mark.parametrize("name", list(REPACKED))
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16, ta.float32], ids=str)
def test_products_whose_operands_are_copied_into_aligned_rows(device, dtype, name):
    sa, sb, va, vb = REPACKED[name]
    ha, da = support.both(support.values_for(dtype, SEED, 41, sa, -1, 1), dtype, device)
    hb, db = support.both(support.values_for(dtype, SEED, 42, sb, -1, 1), dtype, device)
    want = ops.matmul(support.apply_view(ha, va), support.apply_view(hb, vb)).numpy()
    got = ops.matmul(support.apply_view(da, va), support.apply_view(db, vb)).numpy()
    k = support.apply_view(ha, va).shape[-1]
    if dtype is ta.float32: support.assert_close(got, want, 1e-5, k * 2.0 ** -24, f"gemm {dtype} {name}")
    else: support.assert_close(got, want, 2e-3 if dtype is ta.float16 else 2.0 ** -7, 1e-3, f"gemm {dtype} {name}")


@pytest.mark.parametrize("pair", [(ta.int32, ta.float32), (ta.float64, ta.float32), (ta.float16, ta.float32), (ta.float32, ta.bfloat16)],
                         ids=lambda p: f"{p[0]}-{p[1]}")
def test_mixed_gemm(device, pair):
    host, dev, k = operands(pair, "nt_mid", device, -3, 3)
    want, got = ops.matmul(*host), ops.matmul(*dev)
    assert got.dtype is want.dtype
    support.assert_close(got.numpy(), want.numpy(), 1e-5, k * 9 * 2.0 ** -24, f"gemm {pair}")


@pytest.mark.parametrize("layout", ["thousand_square_nt", "thousand_square_tn", "nn_large_tiles_batched", "rank4_rank2_nt_large", "stream_49_rows_long_k_wide"])
@pytest.mark.parametrize("pair", [(ta.int32, ta.float32), (ta.float64, ta.float32), (ta.float16, ta.float32), (ta.float32, ta.bfloat16), (ta.bfloat16, ta.float64),
                                  (ta.int64, ta.float16), (ta.int32, ta.bfloat16)], ids=lambda p: f"{p[0]}-{p[1]}")
def test_large_mixed_gemm_multiplies_converted_copies(device, pair, layout):
    """Pairs of different types with an fp32 / float64 result, large enough that the operands are converted to the result
    type first (in the order of their own strides) and multiplied on the matrix pipe: the same numbers as
    static_cast<D>(a) * static_cast<D>(b) summed (src/cpu/matmul.cpp:36), in a different order."""
    host, dev, k = operands(pair, layout, device, -3, 3)
    want, got = ops.matmul(*host), ops.matmul(*dev)
    assert got.dtype is want.dtype and got.shape == want.shape
    eps = 2.0 ** -53 if want.dtype is ta.float64 else 2.0 ** -24
    support.assert_close(got.numpy(), want.numpy(), 1e-13 if want.dtype is ta.float64 else 1e-5, k * 9 * eps, f"gemm {pair} {layout}")


def test_operand_with_fewer_batch_dims_steps_by_its_own_batch_stride(device):
    """a[3,M,K] x b[2,3,K,N]: the batch coordinate of `a` is looked up right-aligned and multiplied by the stride of
    that same dim.  (The reference multiplies it by the stride at the left-aligned position, src/cpu/matmul.cpp:107-118,
    i.e. steps `a` by its row stride: this is a documented difference, so the expectation here is numpy's.)"""
    a = support.uniform(SEED, 5, (3, 9, 16))
    b = support.uniform(SEED, 6, (2, 3, 16, 11))
    for dtype, rtol, atol in ((ta.float32, 1e-5, 16 * 2.0 ** -24), (ta.float16, 2e-3, 1e-3), (ta.int32, 0, 0)):
        va = np.floor(a * 50) if dtype.is_integral else a
        vb = np.floor(b * 50) if dtype.is_integral else b
        _, da = support.both(va, dtype, device)
        _, db = support.both(vb, dtype, device)
        got = ops.matmul(da, db).numpy().astype(np.float64)
        ra = da.numpy().astype(np.float64)
        rb = db.numpy().astype(np.float64)
        support.assert_close(got, np.matmul(ra, rb), rtol, atol, f"rank 3 x rank 4 {dtype}")
        got = ops.matmul(db.transpose(), da.transpose()).numpy().astype(np.float64)      # [2,3,N,K] x [3,K,M]
        support.assert_close(got, np.matmul(rb.swapaxes(-1, -2), ra.swapaxes(-1, -2)), rtol, atol, f"rank 4 x rank 3 {dtype}")


@pytest.mark.parametrize("shape", [(1024, 2048, 512), (2048, 4096, 256), (512, 4096, 1024), (512, 4096, 4096), (256, 2048, 8192), (4096, 4096, 128), (2304, 8192, 192), (2, 2048, 6144, 64), (25, 512, 1024, 64),
                                   (264, 392, 2048), (2, 136, 784, 2048), (520, 4104, 4096), (512, 2048, 16384)], ids=str)
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_operands_contiguous_along_m_or_n_on_direct_tiles(device, dtype, shape):
    """X . W, X^T . W and X^T . W^T with whole tiles along M and N (the last three shapes: with a last tile that reaches
    past M and N, long K; the last: a long K shared between many workgroups), at sizes that choose each tile of the direct-to-LDS
    kernel (128 x 128, 256 x 128, K shared between two and more workgroups, 256 x 256, more 256 x 256 tiles than compute units
    so that a workgroup walks several, batches): operand tiles kept as k-rows and
    read with the transposing LDS read.  Sums run over k in the same order as for X . W^T, so the four layouts agree
    bit for bit; X . W^T itself is checked against float64 on sampled rows."""
    *batch, m, n, k = shape
    x = support.values_for(dtype, SEED, 5, (*batch, m, k), -1, 1)
    w = support.values_for(dtype, SEED, 6, (*batch, k, n), -1, 1)
    hx, dx = support.both(x, dtype, device)
    _, dxt = support.both(np.ascontiguousarray(np.swapaxes(x, -1, -2)), dtype, device)
    hw, dw = support.both(w, dtype, device)
    _, dwt = support.both(np.ascontiguousarray(np.swapaxes(w, -1, -2)), dtype, device)
    nt = ops.matmul(dx, dwt.transpose(-1, -2)).numpy()
    rows = np.random.default_rng(SEED).choice(m, 32, replace=False)
    exact = np.matmul(hx.numpy().astype(np.float64)[..., rows, :], hw.numpy().astype(np.float64))
    rtol = 2e-3 if dtype is ta.float16 else 2.0 ** -7
    support.assert_close(nt[..., rows, :], exact, rtol, 1e-3 * np.sqrt(k), f"nt {dtype} {shape}")
    for name, a, b in (("nn", dx, dw), ("tn", dxt.transpose(-1, -2), dw), ("tt", dxt.transpose(-1, -2), dwt.transpose(-1, -2))):
        got = ops.matmul(a, b).numpy()
        support.assert_bit_exact(got, nt, f"{name} against nt, {dtype} {shape}")


@pytest.mark.parametrize("shape", [(2048, 14336, 256), (2048, 12288, 192), (2000, 14000, 128), (2048, 12200, 64)], ids=str)
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_tile_widths_between_the_powers_of_two(device, dtype, shape):
    """Extents for which 256 x 224 and 256 x 192 tiles need fewer rounds than 256 x 256 ones, with whole and with ragged
    last tiles along both M and N: X . W^T against float64 on sampled rows (all columns, so every tile column is seen),
    and, where N is a whole number of 256-wide tiles, bit for bit against X . W, which runs 256-wide k-row tiles."""
    m, n, k = shape
    x = support.values_for(dtype, SEED, 7, (m, k), -1, 1)
    w = support.values_for(dtype, SEED, 8, (k, n), -1, 1)
    hx, dx = support.both(x, dtype, device)
    hw, dw = support.both(w, dtype, device)
    _, dwt = support.both(np.ascontiguousarray(w.T), dtype, device)
    nt = ops.matmul(dx, dwt.transpose()).numpy()
    rows = np.concatenate([np.random.default_rng(SEED).choice(m, 30, replace=False), [0, m - 1]])
    exact = np.matmul(hx.numpy().astype(np.float64)[rows, :], hw.numpy().astype(np.float64))
    rtol = 2e-3 if dtype is ta.float16 else 2.0 ** -7
    support.assert_close(nt[rows, :], exact, rtol, 1e-3 * np.sqrt(k), f"nt {dtype} {shape}")
    if n % 256 == 0 and m % 256 == 0:
        support.assert_bit_exact(ops.matmul(dx, dw).numpy(), nt, f"nn against nt, {dtype} {shape}")


def test_integer_valued_fp16_gemm_is_exact(device):
    """Small integers: every product and partial sum is exact in fp32, so any order of summation agrees."""
    a = support.integers(SEED, 3, (192, 320), -4, 4)
    b = support.integers(SEED, 4, (160, 320), -4, 4)
    for dtype in (ta.float16, ta.bfloat16, ta.float32):
        _, da = support.both(a, dtype, device)
        _, db = support.both(b, dtype, device)
        got = ops.matmul(da, db.transpose()).numpy().astype(np.int64)
        want = a @ b.T
        if dtype is ta.bfloat16:
            want = support.types.bfloat16_bits_to_float32(support.types.float32_to_bfloat16_bits(want.astype(np.float32))).astype(np.int64)
        else:
            want = want.astype(np.float16 if dtype is ta.float16 else np.float32).astype(np.int64)
        support.assert_bit_exact(got, want, f"integer-valued {dtype}")


def test_fp32_matmul_512_seed0(device):
    """C = A.B, 512^3, uniform[-1,1) from seed 0: the reference's CPU-runnable configuration."""
    a, b = support.uniform(0, 0, (512, 512)), support.uniform(0, 1, (512, 512))
    (ha, da), (hb, db) = support.both(a, ta.float32, device), support.both(b, ta.float32, device)
    want, got = ops.matmul(ha, hb).numpy(), ops.matmul(da, db).numpy()
    support.assert_close(got, want, 1e-5, 512 * 2.0 ** -24, "fp32 512^3")
    exact = a.astype(np.float64) @ b.astype(np.float64)
    assert np.abs(got - exact).max() <= np.abs(want - exact).max() * 1.5 + 1e-6  # no worse than the sequential sum


@pytest.mark.parametrize("dtype", [ta.float16, ta.float32, ta.int32, ta.float64], ids=str)
def test_operands_whose_inner_stride_is_not_one(device, oracle, dtype):
    """Views with both matrix strides different from 1 (every other column, one half of an interleaved tensor, an
    expanded column) multiply the elements they show: checked against numpy on small integers, where every type is
    exact.  (The reference's CPU path takes the smaller stride to be 1, src/cpu/matmul.cpp:87-94.)"""
    rng = np.random.default_rng(5)
    a = rng.integers(-3, 4, (40, 70)).astype(np.float64)
    b = rng.integers(-3, 4, (70, 50)).astype(np.float64)
    ha, da = support.both(a, dtype, device)
    hb, db = support.both(b, dtype, device)
    index_a, index_b = (slice(3, 35, 2), slice(1, 61, 2)), (slice(10, 40), slice(2, 50, 3))
    want = a[index_a] @ b[index_b]
    for x, y in ((da, db), (ha, hb)):
        np.testing.assert_array_equal(ops.matmul(x[index_a], y[index_b]).numpy().astype(np.float64), want)
    pairs = rng.integers(-3, 4, (16, 24, 2)).astype(np.float64)          # [M, K, 2]: the "real parts" are a stride-2 view
    hp, dp = support.both(pairs, dtype, device)
    w = rng.integers(-3, 4, (24, 8)).astype(np.float64)
    hw, dw = support.both(w, dtype, device)
    for x, y in ((dp, dw), (hp, hw)):
        np.testing.assert_array_equal(ops.matmul(x[:, :, 0], y).numpy().astype(np.float64), pairs[:, :, 0] @ w)
    column = rng.integers(-3, 4, (16, 1)).astype(np.float64)
    hc, dc = support.both(column, dtype, device)
    for x, y in ((dc, dw), (hc, hw)):
        np.testing.assert_array_equal(ops.matmul(x.expand(16, 24), y).numpy().astype(np.float64), np.broadcast_to(column, (16, 24)) @ w)

"""GPU parity of the W4A16 linear kernels against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

import oracle
from tests.gpu_util import assert_close_to_oracle, linear_grid, u32s, w4_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def runtime():
    from llmopt_amd.native import Runtime
    rt = Runtime()
    yield rt
    rt.close()


def run_linear(runtime, x, packed, scale, bias=None, residual=None, name=None):
    m, k = x.shape
    n = packed.shape[0]
    addend = bias if bias is not None else residual
    stride = n if residual is not None else 0
    bx = runtime.buffer_of_bytes(x)
    bw = runtime.buffer_of_bytes(packed)
    bs = runtime.buffer_of_bytes(scale)
    ba = runtime.buffer_of_bytes(addend) if addend is not None else bs
    out = runtime.buffer_of_bytes(np.full((m, n), np.nan, dtype=np.float16))  # NaN sentinel
    if name is None:
        name = "llmopt_w4a16_linear_f16_g64" if m == 1 else "llmopt_w4a16_linear_f16_g64_m4"
    columns = m * n if m == 1 else ((m + 3) // 4) * n
    runtime.dispatch(name, [bx, bw, bs, ba, out],
                     u32s(m, n, k, 1 if addend is not None else 0, stride),
                     grid=(linear_grid(columns), 1, 1), group=(256, 1, 1))
    return out.numpy(np.float16, (m, n))


def every_byte_matrix(rng):
    """64 rows x 256 K values in which every byte value (both nibbles) occurs in every byte lane of
    a weight dword."""
    packed = np.empty((64, 128), dtype=np.uint8)
    for row in range(64):
        values = np.arange(256, dtype=np.uint8)
        rng.shuffle(values)
        # rotate so that byte lane (column % 4) sees another quarter of the values on each row
        packed[row] = np.roll(values, row)[:128] if row % 2 == 0 else np.roll(values, row)[128:]
    return packed


@pytest.mark.parametrize("decoder,name", [(0, "w4_decode_pairs"), (1, "w4_decode_biased")])
def test_product_nibble_decoders_are_bit_exact(runtime, decoder, name):
    """The two decoders every W4A16 kernel uses, over all 256 byte values in all four byte lanes
    of a dword and a spread of fp16 scales: float32 q * s identical to the oracle's, bit for bit."""
    rng = np.random.default_rng(decoder)
    packed = every_byte_matrix(rng)
    for lane in range(4):
        assert len(set(packed[:, lane::4].reshape(-1).tolist())) == 256
    scale = rng.uniform(0.005, 0.02, size=(64, 4)).astype(np.float16)
    scale[0] = [1.0, 2.0 ** -14, 65504.0, 6e-8]  # unit, smallest normal, largest, subnormal
    bw, bs = runtime.buffer_of_bytes(packed), runtime.buffer_of_bytes(scale)
    out = runtime.create_buffer(64 * 256 * 4)
    runtime.dispatch("llmopt_w4_dequant_f32", [bw, bs, out], u32s(64, 256, decoder))
    got = out.numpy(np.float32, (64, 256))
    np.testing.assert_array_equal(got.view(np.uint32), oracle.w4_dequant(packed, scale).view(np.uint32), err_msg=name)
    # and the integers themselves, against arithmetic written here: low nibble = even K, two's complement
    ones = np.ones((64, 4), dtype=np.float16)
    runtime.dispatch("llmopt_w4_dequant_f32", [bw, runtime.buffer_of_bytes(ones), out], u32s(64, 256, decoder))
    integers = out.numpy(np.float32, (64, 256))
    low = (packed & 15).astype(np.int32)
    high = (packed >> 4).astype(np.int32)
    expected = np.stack([low - 16 * (low >= 8), high - 16 * (high >= 8)], axis=-1).reshape(64, 256)
    np.testing.assert_array_equal(integers, expected.astype(np.float32), err_msg=name)


def test_default_dequant_entry_is_bit_exact(runtime):
    rng = np.random.default_rng(0)
    packed = every_byte_matrix(rng)
    scale = rng.uniform(0.005, 0.02, size=(64, 4)).astype(np.float16)
    out = runtime.create_buffer(64 * 256 * 4)
    runtime.dispatch("llmopt_w4_dequant_f32", [runtime.buffer_of_bytes(packed), runtime.buffer_of_bytes(scale), out],
                     u32s(64, 256))
    np.testing.assert_array_equal(out.numpy(np.float32, (64, 256)).view(np.uint32),
                                  oracle.w4_dequant(packed, scale).view(np.uint32))


def test_gemm_staged_weight_is_one_half_rounding_from_exact(runtime):
    """The prefill GEMM keeps half(q * s) in LDS: one rounding per weight.  Over every nibble value
    and every finite positive fp16 scale the staged value is the correctly rounded product, i.e.
    within 2^-11 relative of q * s wherever the product is a normal half, and exact for the
    configurations' scales times powers of two."""
    scales = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16)  # every positive finite half
    rows = (scales.size + 3) // 4
    scale = np.ones(rows * 4, dtype=np.float16)
    scale[:scales.size] = scales
    scale = scale.reshape(rows, 4)
    # each 64-wide group holds the 16 nibble values four times over
    packed = np.tile(np.array([0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE], dtype=np.uint8), (rows, 16))
    out = runtime.create_buffer(rows * 256 * 4)
    runtime.dispatch("llmopt_w4_dequant_f32", [runtime.buffer_of_bytes(packed), runtime.buffer_of_bytes(scale), out],
                     u32s(rows, 256, 2))
    staged = out.numpy(np.float32, (rows, 256)).astype(np.float64)
    exact = oracle.w4_dequant(packed, scale).astype(np.float64)
    with np.errstate(over="ignore"):
        rounded = exact.astype(np.float16).astype(np.float64)  # IEEE round-to-nearest-even, inf on overflow
    np.testing.assert_array_equal(staged, rounded)
    normal = (np.abs(exact) >= 2.0 ** -14) & np.isfinite(rounded)
    relative = np.abs(staged[normal] - exact[normal]) / np.abs(exact[normal])
    assert relative.max() <= 2.0 ** -11
    assert np.all(np.isfinite(staged[np.abs(exact) <= 65504.0]))


def test_reference_fixture_golden_bits(runtime, golden):
    case = golden["w4a16_linear_fixture"]
    packed = np.arange(96, dtype=np.uint8).reshape(3, 32)
    packed[0, 0] = 0x78
    scale = np.array(case["scale"], dtype=np.float16).reshape(3, 1)
    bias = np.array(case["bias"], dtype=np.float16)
    x = np.full((2, 64), 1.0, dtype=np.float16)
    out = run_linear(runtime, x, packed, scale, bias=bias)
    assert out.view(np.uint16).reshape(-1).tolist() == case["expected_output_bits"]


@pytest.mark.parametrize("with_bias", [True, False])
def test_runtime_smoke_is_exact(runtime, golden, with_bias):
    case = golden["w4a16_runtime_smoke"]
    m, n, k = case["m"], case["n"], case["k"]
    packed = np.empty((n, k // 2), dtype=np.uint8)
    packed[0::2] = case["even_row_byte"]
    packed[1::2] = case["odd_row_byte"]
    scale = np.full((n, 1), case["scale"], dtype=np.float16)
    bias = np.arange(n, dtype=np.float16) if with_bias else None
    x = np.ones((m, k), dtype=np.float16)
    out = run_linear(runtime, x, packed, scale, bias=bias)
    expected = oracle.w4a16_linear(x, packed, scale, bias).astype(np.float16)
    np.testing.assert_array_equal(out.view(np.uint16), expected.view(np.uint16))


GEMV_SHAPES = [(1, 1536, 576), (1, 4096, 4096), (2, 512, 4096), (3, 260, 1024), (4, 96, 14336),
               (5, 64, 640), (8, 200, 4096), (8, 33, 14336), (7, 1, 64),
               # many short rows: one and two activation rows on the matrix-core kernel
               (1, 16384, 576), (2, 20008, 1024), (2, 16385, 64)]


@pytest.mark.parametrize("m,n,k", GEMV_SHAPES)
def test_gemv_matches_oracle(runtime, m, n, k):
    rng = np.random.default_rng(1000 * m + n + k)
    x, packed, scale, bias = w4_case(rng, m, n, k, bias=True)
    expected = oracle.w4a16_linear(x, packed, scale, None)
    assert_close_to_oracle(run_linear(runtime, x, packed, scale), expected, f"gemv {m}x{n}x{k}")
    expected_bias = oracle.add(expected, bias.astype(np.float32).reshape(1, -1))
    assert_close_to_oracle(run_linear(runtime, x, packed, scale, bias=bias), expected_bias,
                           f"gemv+bias {m}x{n}x{k}")


@pytest.mark.parametrize("m", [4, 17])
def test_gemv_residual_epilogue(runtime, m):
    rng = np.random.default_rng(5)
    n, k = 576, 1536
    x, packed, scale, _ = w4_case(rng, m, n, k)
    residual = rng.standard_normal((m, n)).astype(np.float16)
    expected = oracle.add(oracle.w4a16_linear(x, packed, scale, None), residual.astype(np.float32))
    assert_close_to_oracle(run_linear(runtime, x, packed, scale, residual=residual), expected,
                           "gemv+residual")


# up to 128 rows with small weights run the matrix-core GEMV once per group of 8 rows
GEMM_SHAPES = [(9, 64, 64), (16, 128, 128), (24, 576, 1536), (31, 100, 576), (32, 1536, 576),
               (32, 96, 14336), (33, 64, 576), (64, 576, 1536), (100, 29, 192), (128, 192, 576), (129, 64, 576), (128, 256, 512), (130, 300, 1024),
               (512, 128, 4096), (200, 130, 256), (140, 260, 768), (512, 4096, 256),
               # K that is not a whole number of four-step passes on the four-stage small tiles: 9, 1 and 5 steps
               (300, 576, 576), (2048, 192, 64), (513, 200, 320)]


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_gemm_matches_oracle(runtime, m, n, k):
    rng = np.random.default_rng(7 * m + n + k)
    x, packed, scale, bias = w4_case(rng, m, n, k, bias=True)
    expected = oracle.w4a16_linear(x, packed, scale, bias)
    assert_close_to_oracle(run_linear(runtime, x, packed, scale, bias=bias), expected,
                           f"gemm {m}x{n}x{k}")


def test_gemm_linearity_at_full_size(runtime):
    """M=2048, K=4096, N=4096: too large for the serial oracle, so check sampled
    output columns against it and linearity (2x activation -> 2x output, exact in fp16)."""
    rng = np.random.default_rng(77)
    m, n, k = 2048, 4096, 4096
    x, packed, scale, _ = w4_case(rng, m, n, k)
    out = run_linear(runtime, x, packed, scale)
    doubled = run_linear(runtime, (x.astype(np.float32) * 2).astype(np.float16), packed, scale)
    base, twice = out.astype(np.float32), doubled.astype(np.float32)
    normal = np.abs(base) >= 2.0 ** -13  # doubling is exact in fp16 except from the subnormal range
    np.testing.assert_array_equal(twice[normal], 2 * base[normal])
    assert normal.mean() > 0.99
    columns = rng.choice(n, size=24, replace=False)
    rows = rng.choice(m, size=64, replace=False)
    expected = oracle.w4a16_linear(x[rows], packed[columns], scale[columns], None)
    assert_close_to_oracle(out[np.ix_(rows, columns)], expected, "gemm sampled")


def qkv_params(m, k, nq, nk, nv):
    return u32s(m, k, nq, nk, nv)


@pytest.mark.parametrize("m", [1, 4, 8, 12, 32, 40, 130])
def test_qkv_linear(runtime, m):
    rng = np.random.default_rng(31 + m)
    k, sizes = 576, (576, 192, 192)
    x = rng.standard_normal((m, k)).astype(np.float16)
    mats = [w4_case(rng, 1, n, k)[1:3] for n in sizes]
    buffers = [runtime.buffer_of_bytes(x)]
    for packed, scale in mats:
        buffers += [runtime.buffer_of_bytes(packed), runtime.buffer_of_bytes(scale)]
    outs = [runtime.buffer_of_bytes(np.full((m, n), np.nan, dtype=np.float16)) for n in sizes]
    name = "llmopt_w4a16_qkv_linear_f16_g64" + ("" if m == 1 else "_m4")
    runtime.dispatch(name, buffers + outs, qkv_params(m, k, *sizes),
                     grid=(linear_grid(m * sum(sizes)), 1, 1), group=(256, 1, 1))
    for (packed, scale), out, n in zip(mats, outs, sizes):
        assert_close_to_oracle(out.numpy(np.float16, (m, n)),
                               oracle.w4a16_linear(x, packed, scale, None), f"qkv n={n}")


@pytest.mark.parametrize("m,k", [(1, 576), (2, 576), (1, 2048), (2, 64), (3, 576), (8, 576), (40, 576), (1, 4096),
                                 (130, 576), (4, 4096), (5, 64), (8, 14336), (128, 1536), (32, 576), (17, 1536)])
def test_normalising_qkv_and_swiglu_entries(runtime, m, k):
    """The extension entries that take the raw rows and the norm weight: against the oracle's
    RMSNorm (rounded to half, as the separate kernel stores it) followed by the projections, and
    against the two launches they stand for - to a few half roundings where the projection kernel
    normalises itself (its mean square is summed in another order), bit for bit where the entry
    runs the two kernels."""
    import struct
    rng = np.random.default_rng(500 + 7 * m + k)
    sizes, n = (192, 64, 64), 256
    epsilon = 1e-5
    x = (rng.standard_normal((m, k)) * 3.0).astype(np.float16)
    gain = rng.uniform(0.5, 1.5, size=k).astype(np.float16)
    mats = [w4_case(rng, 1, width, k)[1:3] for width in sizes]
    _, gate_w, gate_s, _ = w4_case(rng, 1, n, k)
    _, up_w, up_s, _ = w4_case(rng, 1, n, k)
    bx, bg = runtime.buffer_of_bytes(x), runtime.buffer_of_bytes(gain)
    weights = []
    for packed, scale in mats:
        weights += [runtime.buffer_of_bytes(packed), runtime.buffer_of_bytes(scale)]
    ffn_weights = [runtime.buffer_of_bytes(a) for a in (gate_w, gate_s, up_w, up_s)]
    suffix = "" if m == 1 else "_m4"
    rows_grid = (((m + 7) // 8) * 256, 1, 1)
    blank = lambda width: runtime.buffer_of_bytes(np.full((m, width), np.nan, dtype=np.float16))

    # the two launches
    normed = blank(k)
    runtime.dispatch("llmopt_rms_norm_f16_simd", [bx, bg, normed], struct.pack("<IIf", m, k, epsilon),
                     grid=rows_grid, group=(256, 1, 1))
    two = [blank(width) for width in sizes]
    runtime.dispatch("llmopt_w4a16_qkv_linear_f16_g64" + suffix, [normed, *weights, *two], qkv_params(m, k, *sizes),
                     grid=(linear_grid(m * sum(sizes)), 1, 1), group=(256, 1, 1))
    ffn_params = u32s(m, n, k) + struct.pack("<f", epsilon)
    ffn_normed = blank(k)
    runtime.dispatch("llmopt_w4a16_swiglu_rms_f16_g64", [bx, bg, ffn_normed], ffn_params,
                     grid=(m * 256, 1, 1), group=(256, 1, 1))
    two_product = blank(n)
    runtime.dispatch("llmopt_w4a16_dual_swiglu_f16_g64" + suffix, [ffn_normed, *ffn_weights, two_product], ffn_params,
                     grid=(linear_grid(m * n), 1, 1), group=(256, 1, 1))

    # one launch each
    one = [blank(width) for width in sizes]
    runtime.dispatch("llmopt_rms_w4a16_qkv_linear_f16_g64", [bx, bg, *weights, *one],
                     qkv_params(m, k, *sizes) + struct.pack("<f", epsilon),
                     grid=(linear_grid(m * sum(sizes)), 1, 1), group=(256, 1, 1))
    one_product = blank(n)
    runtime.dispatch("llmopt_rms_w4a16_dual_swiglu_f16_g64", [bx, bg, *ffn_weights, one_product], ffn_params,
                     grid=(linear_grid(m * n), 1, 1), group=(256, 1, 1))

    # one or two rows: K of one chunk; 3..32 rows: the matrix-core GEMV when one workgroup covers K
    in_kernel = (m <= 2 and k <= 2048) or (3 <= m <= 32 and k <= 4096)
    normalised = oracle.rms_norm(x, gain, epsilon).astype(np.float16)
    for (packed, scale), got, reference, width in zip(mats, one, two, sizes):
        got = got.numpy(np.float16, (m, width))
        assert_close_to_oracle(got, oracle.w4a16_linear(normalised, packed, scale, None), f"rms+qkv n={width}")
        if in_kernel:
            assert_close_to_oracle(got, reference.numpy(np.float16, (m, width)).astype(np.float32), "rms+qkv vs two")
        else:
            np.testing.assert_array_equal(got.view(np.uint16), reference.numpy(np.uint16, (m, width)))
    got = one_product.numpy(np.float16, (m, n))
    expected = oracle.silu_mul(oracle.w4a16_linear(normalised, gate_w, gate_s, None),
                               oracle.w4a16_linear(normalised, up_w, up_s, None))
    assert_close_to_oracle(got, expected, "rms+dual swiglu")
    if in_kernel:
        assert_close_to_oracle(got, two_product.numpy(np.float16, (m, n)).astype(np.float32), "rms+dual vs two")
    else:
        np.testing.assert_array_equal(got.view(np.uint16), two_product.numpy(np.uint16, (m, n)))


@pytest.mark.parametrize("m", [1, 2, 4, 8, 9, 32, 48, 136, 600])
def test_swiglu_ffn_chain(runtime, m):
    """dual-SwiGLU then down+residual, the two W4A16 stages of the reference's
    FFN macro-op; the intermediate product is rounded to f16 between stages
    (lib/metal_w4a16_source.ml:574-575)."""
    import struct
    rng = np.random.default_rng(91 + m)
    k, n = 576, 1536
    x = rng.standard_normal((m, k)).astype(np.float16)
    _, gate_w, gate_s, _ = w4_case(rng, 1, n, k)
    _, up_w, up_s, _ = w4_case(rng, 1, n, k)
    _, down_w, down_s, _ = w4_case(rng, 1, k, n)
    residual = rng.standard_normal((m, k)).astype(np.float16)
    params = u32s(m, n, k) + struct.pack("<f", 1e-5)
    suffix = "" if m == 1 else "_m4"
    product = runtime.buffer_of_bytes(np.full((m, n), np.nan, dtype=np.float16))
    runtime.dispatch("llmopt_w4a16_dual_swiglu_f16_g64" + suffix,
                     [runtime.buffer_of_bytes(x), runtime.buffer_of_bytes(gate_w),
                      runtime.buffer_of_bytes(gate_s), runtime.buffer_of_bytes(up_w),
                      runtime.buffer_of_bytes(up_s), product], params,
                     grid=(linear_grid(m * n), 1, 1), group=(256, 1, 1))
    gate = oracle.w4a16_linear(x, gate_w, gate_s, None)
    up = oracle.w4a16_linear(x, up_w, up_s, None)
    expected_product = oracle.silu_mul(gate, up)
    got_product = product.numpy(np.float16, (m, n))
    assert_close_to_oracle(got_product, expected_product, "dual swiglu")
    output = runtime.buffer_of_bytes(np.full((m, k), np.nan, dtype=np.float16))
    runtime.dispatch("llmopt_w4a16_down_add_f16_g64" + suffix,
                     [product, runtime.buffer_of_bytes(down_w), runtime.buffer_of_bytes(down_s),
                      runtime.buffer_of_bytes(residual), output], params,
                     grid=(linear_grid(m * k), 1, 1), group=(256, 1, 1))
    expected = oracle.add(oracle.w4a16_linear(got_product, down_w, down_s, None),
                          residual.astype(np.float32))
    assert_close_to_oracle(output.numpy(np.float16, (m, k)), expected, "down+residual")


# ---- the benchmark's own cells, at full size ------------------------------------------------
# Every kernel instantiation the measured configurations select: the single-row ring kernel at
# K >= 8192, the two-row variant whose activation fills 57 KB of LDS, the persistent 768-workgroup
# grids at N = 14336 and the K = 14336 split over workgroups.  The oracle runs the whole matrix.
SWEEP_CELLS = [(m, n, k) for m in (1, 2, 4, 8) for k, n in ((4096, 4096), (4096, 14336), (14336, 4096))]


@pytest.mark.parametrize("m,n,k", SWEEP_CELLS)
def test_gemv_sweep_cell_at_full_size(runtime, m, n, k):
    rng = np.random.default_rng(31 * m + n + 7 * k)
    x, packed, scale, bias = w4_case(rng, m, n, k, bias=True)
    print(f"gemv sweep cell m={m} n={n} k={k}", flush=True)
    expected = oracle.w4a16_linear(x, packed, scale, None)
    assert_close_to_oracle(run_linear(runtime, x, packed, scale), expected, f"gemv cell {m}x{n}x{k}")
    if m in (1, 2, 8):  # the addend path of the same grids
        expected_bias = oracle.add(expected, bias.astype(np.float32).reshape(1, -1))
        assert_close_to_oracle(run_linear(runtime, x, packed, scale, bias=bias), expected_bias,
                               f"gemv cell+bias {m}x{n}x{k}")


# The one-workgroup-per-CU GEMV on the 4x4x4 matrix-core blocks (1..4 rows, K = 4096 / 14336):
# every (row quads per wave, waves, ring) choice of its launcher, a last workgroup that is only
# partly there (N = 4100, 9004), three rows inside a four-row staging, and both addend kinds.
QUAD_CELLS = [(3, 4096, 4096, "bias"), (2, 4100, 4096, "residual"), (4, 6144, 4096, "bias"),
              (3, 9004, 4096, "residual"), (2, 11008, 4096, None), (4, 14336, 4096, "residual"),
              (1, 4100, 14336, "bias"), (3, 6144, 14336, "residual"), (4, 4096, 14336, "bias"),
              (2, 9004, 14336, None), (4, 3072, 14336, None),
              # three and four rows of K = 14336 beyond N = 8192 leave the quad kernel (no instantiation without spills)
              (3, 9004, 14336, "bias"),
              # three and four rows at any K that is a multiple of 128 up to 8192 (the instantiations cut for rows
              # of 8192 values, the walk over K stopping at the row's end, the last 512-wide range partly
              # there): short and long rings, one and two quads per wave, the shortest and the longest rows;
              # one and two rows of such K, and longer rows, run the kernels of w4a16_gemv.hip / _mfma.hip
              (1, 8192, 8192, None), (4, 8192, 8192, "residual"), (1, 5120, 5120, "bias"), (4, 5120, 5120, None),
              (2, 4096, 2048, "residual"), (3, 12288, 2560, None), (4, 3100, 7680, "bias"), (1, 4096, 11264, None),
              (2, 9004, 16384, "residual"), (1, 3072, 16384, "bias"), (2, 4096, 10240, None),
              # N beyond one round of workgroups (28672 rows: two rounds; 49152: four)
              (1, 28672, 4096, None), (4, 28672, 4096, "residual"), (2, 49152, 2048, "bias"), (1, 30000, 14336, None),
              # a last K range that is partly there (11008 = 21.5 ranges, 2176 = 4.25, 5248 = 10.25, 16256 = 31.75)
              (2, 4096, 11008, "bias"), (1, 11008, 11008, None), (4, 4096, 2176, "residual"), (3, 5120, 5248, None),
              (4, 9004, 7808, "bias"), (2, 3072, 16256, None),
              (3, 4096, 2048, "bias"), (4, 8192, 4096 + 128, None), (3, 28672, 8192, "residual"),
              # K not a multiple of 128, four rows beyond 8192
              (4, 4096, 4160, "bias"), (4, 4096, 11264, None)]


@pytest.mark.parametrize("m,n,k,addend", QUAD_CELLS)
def test_gemv_quad_kernel_shapes(runtime, m, n, k, addend):
    rng = np.random.default_rng(13 * m + n + 3 * k)
    x, packed, scale, bias = w4_case(rng, m, n, k, bias=True)
    residual = rng.standard_normal((m, n)).astype(np.float16)
    print(f"gemv quad cell m={m} n={n} k={k} addend={addend}", flush=True)
    expected = oracle.w4a16_linear(x, packed, scale, None)
    if addend == "bias":
        expected = oracle.add(expected, bias.astype(np.float32).reshape(1, -1))
        got = run_linear(runtime, x, packed, scale, bias=bias)
    elif addend == "residual":
        expected = oracle.add(expected, residual.astype(np.float32))
        got = run_linear(runtime, x, packed, scale, residual=residual)
    else:
        got = run_linear(runtime, x, packed, scale)
    assert_close_to_oracle(got, expected, f"gemv quad {m}x{n}x{k} {addend}")


def tile_covering_sample(rng, extent, block):
    """One random index out of every `block` consecutive ones: every tile of a tiled kernel is hit."""
    starts = np.arange(0, extent, block)
    return np.minimum(starts + rng.integers(0, block, size=starts.size), extent - 1)


# (384, 19200, 512): three row tiles of 128 pad less than two of 256, and 225 tiles fill the device: 128 x 256 tiles
PREFILL_CELLS = [(512, 4096, 4096), (512, 14336, 4096), (2048, 4096, 4096), (2048, 14336, 4096), (384, 19200, 512)]


@pytest.mark.parametrize("m,n,k", PREFILL_CELLS)
def test_gemm_prefill_cell_at_full_size(runtime, m, n, k):
    """The measured prefill shapes (128x128 with split K, 256x128 and 256x256 workgroup tiles) and one
    that takes 128x256 tiles.  Three checks:
    the oracle on a sample with one row out of every 32 and one column out of every 64 (every
    workgroup tile and every wave tile is hit); the sum over rows of every output column against
    the oracle applied to the summed activation (touches every output element); and linearity."""
    rng = np.random.default_rng(3 * m + n + k)
    x, packed, scale, _ = w4_case(rng, m, n, k)
    print(f"gemm prefill cell m={m} n={n} k={k}", flush=True)
    out = run_linear(runtime, x, packed, scale)
    rows = tile_covering_sample(rng, m, 32)
    columns = tile_covering_sample(rng, n, 64)
    expected = oracle.w4a16_linear(x[rows], packed[columns], scale[columns], None)
    assert_close_to_oracle(out[np.ix_(rows, columns)], expected, f"gemm cell sampled {m}x{n}x{k}")
    # column sums: sum_r y[r, c] = (sum_r x[r]) . w[c]; fp16 rounding of the m outputs averages out
    summed = x.astype(np.float64).sum(axis=0, keepdims=True).astype(np.float32)
    expected_sums = oracle.w4a16_linear(summed, packed, scale, None).astype(np.float64).reshape(-1)
    got_sums = out.astype(np.float64).sum(axis=0)
    error = np.linalg.norm(got_sums - expected_sums) / np.linalg.norm(expected_sums)
    assert error <= 1e-3, f"column sums differ from the oracle: rel-L2 {error:.3e}"
    doubled = run_linear(runtime, (x.astype(np.float32) * 2).astype(np.float16), packed, scale)
    base, twice = out.astype(np.float32), doubled.astype(np.float32)
    normal = np.abs(base) >= 2.0 ** -13
    np.testing.assert_array_equal(twice[normal], 2 * base[normal])


@pytest.mark.parametrize("m", [512, 2048])
def test_dual_swiglu_prefill_cell_at_full_size(runtime, m):
    """silu(gate) * up at K = 4096, N = 14336: tile-covering sample against the oracle, and every
    output element against the two plain projections of the same launch shape combined on the
    host (their own parity is the test above)."""
    import struct
    n, k = 14336, 4096
    rng = np.random.default_rng(40 + m)
    x = rng.standard_normal((m, k)).astype(np.float16)
    _, gate_w, gate_s, _ = w4_case(rng, 1, n, k)
    _, up_w, up_s, _ = w4_case(rng, 1, n, k)
    print(f"dual swiglu prefill cell m={m} n={n} k={k}", flush=True)
    product = runtime.buffer_of_bytes(np.full((m, n), np.nan, dtype=np.float16))
    runtime.dispatch("llmopt_w4a16_dual_swiglu_f16_g64_m4",
                     [runtime.buffer_of_bytes(x), runtime.buffer_of_bytes(gate_w), runtime.buffer_of_bytes(gate_s),
                      runtime.buffer_of_bytes(up_w), runtime.buffer_of_bytes(up_s), product],
                     u32s(m, n, k) + struct.pack("<f", 1e-5),
                     grid=(linear_grid(((m + 3) // 4) * n), 1, 1), group=(256, 1, 1))
    got = product.numpy(np.float16, (m, n))
    rows = tile_covering_sample(rng, m, 32)
    columns = tile_covering_sample(rng, n, 64)
    gate = oracle.w4a16_linear(x[rows], gate_w[columns], gate_s[columns], None)
    up = oracle.w4a16_linear(x[rows], up_w[columns], up_s[columns], None)
    assert_close_to_oracle(got[np.ix_(rows, columns)], oracle.silu_mul(gate, up), f"dual swiglu cell m={m}")
    # everywhere: against silu(gate) * up of the plain projections (fp16 outputs, so a few roundings apart)
    gate_all = run_linear(runtime, x, gate_w, gate_s).astype(np.float64)
    up_all = run_linear(runtime, x, up_w, up_s).astype(np.float64)
    combined = gate_all / (1.0 + np.exp(-gate_all)) * up_all
    assert_close_to_oracle(got, combined.astype(np.float32), f"dual swiglu cell vs projections m={m}",
                           rel_l2_tol=2e-3)


@pytest.mark.parametrize("use_graph", [False, True, 2, 4])
def test_profiled_commit_of_independent_linears(runtime, use_graph):
    """The measuring commit (host launches, one graph, a graph of concurrent branches the launches
    are dealt onto by their bytes) leaves what a plain commit leaves.  Among the launches: two
    that split K over workgroups and share the context's workspace and arrival counters (8 rows,
    K = 14336), which stay in recorded order on one branch."""
    rng = np.random.default_rng(77)
    shapes = [(1, 512, 4096), (8, 256, 14336), (4, 1024, 576), (2, 4096, 4096), (8, 320, 14336), (3, 64, 1536),
              (8, 1536, 576), (1, 2048, 4096)]
    cases = []
    for m, n, k in shapes:
        x, packed, scale, _ = w4_case(rng, m, n, k)
        cases.append((m, n, k, x, packed, scale, runtime.buffer_of_bytes(x), runtime.buffer_of_bytes(packed),
                      runtime.buffer_of_bytes(scale)))

    def record(batch, outputs):
        for (m, n, k, _, _, _, bx, bw, bs), out in zip(cases, outputs):
            name = "llmopt_w4a16_linear_f16_g64" if m == 1 else "llmopt_w4a16_linear_f16_g64_m4"
            columns = m * n if m == 1 else ((m + 3) // 4) * n
            batch.dispatch(name, [bx, bw, bs, bs, out], u32s(m, n, k, 0, 0),
                           grid=(linear_grid(columns), 1, 1), group=(256, 1, 1))

    def fresh_outputs():
        return [runtime.buffer_of_bytes(np.full((m, n), np.nan, dtype=np.float16)) for m, n, *_ in cases]

    plain = fresh_outputs()
    batch = runtime.begin_batch()
    record(batch, plain)
    batch.commit()
    measured = fresh_outputs()
    batch = runtime.begin_batch()
    record(batch, measured)
    assert batch.commit_profiled(repeats=2, use_graph=use_graph) > 0.0
    for (m, n, k, x, packed, scale, *_), first, second in zip(cases, plain, measured):
        expected = first.numpy(np.float16, (m, n))
        assert np.array_equal(second.numpy(np.float16, (m, n)).view(np.uint16), expected.view(np.uint16)), (m, n, k)
        assert_close_to_oracle(expected, oracle.w4a16_linear(x, packed, scale, None), f"linear {m}x{n}x{k}")

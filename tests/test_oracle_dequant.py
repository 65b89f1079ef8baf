"""The numpy restatement of the block-FP8 checkpoint dequantizer against the reference's own
known-answer tests (tests/coverage_test/quantization/test_coverage_hf_checkpoint_dequant.py:210-316;
the vectors below are that file's inputs and expected outputs)."""
import numpy as np
import pytest

from oracle import pf8_oracle as O

E4M3_ONE, UE8M0_ONE = 0x38, 127


def test_e4m3_decodes_zero_subnormal_normal_max_and_nan():
    q = np.array([[0x00, 0x01, E4M3_ONE, 0x7E, 0xFE, 0x7F]], dtype=np.uint8)
    s = np.array([[UE8M0_ONE]], dtype=np.uint8)
    out = O.block_dequant(q, s, "ue8m0", (0, 1), (1, 6))
    np.testing.assert_array_equal(out[0, :5], [0.0, 2.0**-9, 1.0, 448.0, -448.0])
    assert np.isnan(out[0, 5])


def test_ue8m0_scale_codes_decode_to_powers_of_two():
    q = np.full((1, 5), E4M3_ONE, dtype=np.uint8)
    s = np.array([[125, 126, 127, 128, 129]], dtype=np.uint8)
    np.testing.assert_array_equal(O.block_dequant(q, s, "ue8m0", (0, 1), (1, 1)), [[0.25, 0.5, 1.0, 2.0, 4.0]])


def test_ue8m0_table_ends():
    """checkpoint_dequant.py:93: code 0 is 2^-127 (an fp32 subnormal), code 255 is +inf."""
    t = O.ue8m0_table()
    assert t[0] == np.float32(2.0**-127) and t[0] > 0 and np.isinf(t[255]) and t[254] == np.float32(2.0**127)


def test_int8_storage_is_reinterpreted_as_unsigned_codes():
    q = np.array([[E4M3_ONE, -2]], dtype=np.int8)       # -2 is the byte 0xFE
    s = np.full((1, 2), UE8M0_ONE, dtype=np.uint8)
    np.testing.assert_array_equal(O.block_dequant(q, s, "ue8m0", (0, 1), (1, 1)), [[1.0, -448.0]])


def test_block_scales_are_broadcast_across_each_block():
    q = np.full((2, 4), E4M3_ONE, dtype=np.uint8)
    s = np.array([[127, 128]], dtype=np.uint8)
    np.testing.assert_array_equal(O.block_dequant(q, s, "ue8m0", (0, 1), (2, 2)), [[1, 1, 2, 2], [1, 1, 2, 2]])


def test_partial_trailing_block_is_cropped():
    q = np.full((3, 3), E4M3_ONE, dtype=np.uint8)
    s = np.array([[127, 128], [129, 130]], dtype=np.uint8)
    np.testing.assert_array_equal(O.block_dequant(q, s, "ue8m0", (0, 1), (2, 2)), [[1, 1, 2], [1, 1, 2], [4, 4, 8]])


def test_scale_grid_and_rank_mismatch_are_rejected():
    q = np.full((4, 4), E4M3_ONE, dtype=np.uint8)
    with pytest.raises(ValueError, match="Invalid scale grid shape"):
        O.block_dequant(q, np.full((1, 2), 127, dtype=np.uint8), "ue8m0", (0, 1), (2, 2))
    with pytest.raises(ValueError, match="Scale rank must match"):
        O.block_dequant(q, np.full((4,), 127, dtype=np.uint8), "ue8m0", (0, 1), (2, 2))


def test_float_scales_and_bf16_output_match_the_128x128_weight_dequant():
    """The fp32-scale 128x128 case is the C oracle's weight_dequant (kernel.py:100-118)."""
    rng = np.random.default_rng(11)
    q = rng.integers(0, 256, size=(256, 384), dtype=np.uint8)
    q[(q & 0x7F) == 0x7F] = 0x10
    s = rng.uniform(1e-3, 2.0, size=(2, 3)).astype(np.float32)
    np.testing.assert_array_equal(O.block_dequant(q, s, "float32", (0, 1), (128, 128), out="bf16"), O.weight_dequant(q, s))


def test_scales_to_ue8m0_inverts_the_decode_table_over_every_finite_exponent():
    # the table is pinned by the reference's vectors above (code 126 -> 0.5, 127 -> 1, 128 -> 2, 255 -> inf)
    codes = np.arange(1, 255, dtype=np.uint8)
    scales = O.decode_scales(codes, "ue8m0")
    assert np.array_equal(O.scales_to_ue8m0(scales), codes)
    assert O.scales_to_ue8m0(np.array([1.0, 0.5, 2.0 ** -20], np.float32)).tolist() == [127, 126, 107]
    for bad in (0.75, -1.0, 3.0):
        with pytest.raises(ValueError):
            O.scales_to_ue8m0(np.array([bad], np.float32))


def test_pow2_quantizer_scales_are_exact_ue8m0_codes():
    # what the GEMM with exponent-byte scales relies on: a pow2 scale survives the byte round trip
    rng = np.random.default_rng(3)
    x = O.f32_to_bf16_bits(rng.standard_normal((4, 256)).astype(np.float32) * 3.0)
    _, s = O.quant_1x128(x, 0, pow2=True)
    assert np.array_equal(O.decode_scales(O.scales_to_ue8m0(s), "ue8m0"), s)

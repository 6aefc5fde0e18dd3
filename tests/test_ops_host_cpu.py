"""Host-side logic of torchtitan_amd.ops that needs no GPU: operand pitches, shape gates."""
import pytest
import torch

from torchtitan_amd import ops
from torchtitan_amd.ops import MXData, MX_SCALES_MFMA, MX_SCALES_ROWMAJOR


def _codes(rows, cols, pad=0):
    return torch.zeros((rows, cols + pad), dtype=torch.uint8)[:, :cols]


def test_common_pitch_keeps_one_pitch_and_copies_when_they_differ():
    a, b = _codes(64, 256, 128), _codes(32, 256, 128)
    (ra, rb), ld = ops._common_pitch(a, b)
    assert ld == 384 and ra.data_ptr() == a.data_ptr() and rb.data_ptr() == b.data_ptr()
    # dense operands stay as they are
    (ra, rb), ld = ops._common_pitch(_codes(64, 256), _codes(32, 256))
    assert ld == 256 and ra.is_contiguous() and rb.is_contiguous()
    # differing pitches: dense copies of both
    (ra, rb), ld = ops._common_pitch(a, _codes(32, 256))
    assert ld == 256 and ra.is_contiguous() and rb.is_contiguous() and ra.data_ptr() != a.data_ptr()
    # a pitch the persistent kernel does not take (not a multiple of 128) unless the caller allows it
    c, d = _codes(64, 256, 16), _codes(32, 256, 16)
    (rc, rd), ld = ops._common_pitch(c, d)
    assert ld == 256 and rc.is_contiguous()
    (rc, rd), ld = ops._common_pitch(c, d, multiple=16)
    assert ld == 272 and rc.data_ptr() == c.data_ptr()
    # a transposed view is not an operand as it stands
    t = torch.zeros((256, 64), dtype=torch.uint8).t()
    (rt, _), ld = ops._common_pitch(t, _codes(32, 256))
    assert rt.is_contiguous() and ld == 256


def test_code_rows_and_pitch_rule():
    c = ops._code_rows(96, 160, 128, "cpu")
    assert c.shape == (96, 160) and c.stride() == (288, 1)
    s = ops._code_rows(96, 160, 128, "cpu", stack=2)
    assert s.shape == (2, 96, 160) and s.stride() == (96 * 288, 288, 1)
    assert ops._code_rows(96, 160, 0, "cpu").is_contiguous()
    assert ops._pitch_ok(128) == 128 and ops._pitch_ok(16) == 16
    assert ops._pitch_ok(0) == 0 and ops._pitch_ok(8) == 0 and ops._pitch_ok(-128) == 0


def test_unpadded_output_gate():
    def data(rows, cols, order, stack=0):
        shape = (stack, rows, cols) if stack else (rows, cols)
        return MXData(torch.zeros(shape, dtype=torch.uint8), torch.zeros(1, dtype=torch.uint8), order)

    a, b = data(256, 256, MX_SCALES_MFMA), data(128, 256, MX_SCALES_MFMA, stack=4)
    assert ops.rows_out_supported(a, b)
    assert ops.rows_out_supported(a, b, a, b)
    assert not ops.rows_out_supported(a, b, a, None)                                  # half a second operand set
    assert not ops.rows_out_supported(data(256, 256, MX_SCALES_ROWMAJOR), b)          # row-major scales
    assert not ops.rows_out_supported(data(256, 160, MX_SCALES_MFMA), data(128, 160, MX_SCALES_MFMA, stack=4))  # K % 128
    assert not ops.rows_out_supported(data(240, 256, MX_SCALES_MFMA), b)              # T % 32
    assert not ops.rows_out_supported(a, data(128, 256, MX_SCALES_MFMA, stack=ops.FAST_MAX_GROUPS + 1))
    with pytest.raises(ValueError):
        ops.mx_grouped_gemm_2d3d_rows_out(data(256, 256, MX_SCALES_ROWMAJOR), b, torch.zeros(4, dtype=torch.int32),
                                          torch.zeros(4, dtype=torch.int32), 200)
    with pytest.raises(ValueError):  # more output rows than padded rows
        ops.mx_grouped_gemm_2d3d_rows_out(a, b, torch.zeros(4, dtype=torch.int32), torch.zeros(4, dtype=torch.int32), 300)
    with pytest.raises(ValueError):  # int64 group ends
        ops.mx_grouped_gemm_2d3d_rows_out(a, b, torch.zeros(4, dtype=torch.int64), torch.zeros(4, dtype=torch.int32), 200)


def test_block_pitch_is_for_training_steps_without_cached_weight_casts():
    from torchtitan_amd.mx_blocks import block_pitch_pad
    from torchtitan_amd.mx_tensor import MXFP8Config

    cfg = MXFP8Config()
    assert block_pitch_pad(cfg, True, True) == ops.CODE_PITCH_PAD
    assert block_pitch_pad(cfg, True, False) == 0 and block_pitch_pad(cfg, False, True) == 0
    cached = MXFP8Config(cache_weight_casts=True)
    assert block_pitch_pad(cached, True, True) == 0

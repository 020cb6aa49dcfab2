"""GPU parity of the checkpoint -> engine weight converters, through the C ABI, against the
CPU oracle (bit-exact: the outputs are bytes)."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from deepstrix_amd import capi, dispatch
from deepstrix_amd.capi import FMT_Q8_0, SRC_BF16, SRC_F32, SRC_F8E4M3
from oracle import ref

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _convert(src, scale, dtype, split):
    out, inn = src.shape
    dst = torch.zeros(out * (inn // 32) * 34, dtype=torch.uint8, device="cuda")
    dispatch.q8_0_weights_from_hf(dst, dev(src), None if scale is None else dev(scale), dtype,
                                  out, inn, split_rows=split)
    torch.cuda.synchronize()
    return dst.cpu().numpy()


@pytest.mark.parametrize("out,inn,br,bc", [(96, 192, 32, 64), (64, 96, 32, 32), (128, 7168, 32, 32),
                                           (40, 160, 8, 5)])
def test_fp8_checkpoint_to_q8_0_bit_exact(out, inn, br, bc):
    rng = np.random.default_rng(out * 7 + inn)
    codes = rng.integers(0, 256, (out, inn), dtype=np.uint8)    # NaN codes 0x7F / 0xFF included
    scale = rng.integers(100, 150, (out // br, inn // bc), dtype=np.uint8)
    scale[0, 0] = 255
    ggml = ref.q8_0_from_hf(codes, scale, ref.SRC_F8E4M3)
    assert np.array_equal(_convert(codes, scale, SRC_F8E4M3, False), ggml)
    rows = ref.q8_0_repack_rows(ggml, out, inn // 32)
    got = _convert(codes, scale, SRC_F8E4M3, True)
    assert np.array_equal(got, rows)
    # the engine reads what was written: dequantized rows equal the oracle's
    y = torch.zeros((out, inn), dtype=torch.float32, device="cuda")
    dispatch.dequant_rows(FMT_Q8_0, y, dev(got), out, inn)
    assert np.array_equal(y.cpu().numpy().view(np.uint32),
                          ref.q8_0_dequant_rows(rows, out, inn).view(np.uint32))


@pytest.mark.parametrize("inn", [96, 1408, 2048])   # 3 (odd), 44 and 64 blocks per row
def test_bf16_and_f32_checkpoint_to_q8_0_bit_exact(inn):
    rng = np.random.default_rng(inn)
    x = (rng.standard_normal((24, inn)) * 0.02).astype(np.float32)
    x[3, 32:64] = 0.0
    x[5, 0] = 1e30
    bits = torch.from_numpy(x).bfloat16().view(torch.int16).numpy().view(np.uint16)
    for src, dt, rdt in ((x, SRC_F32, ref.SRC_F32), (bits, SRC_BF16, ref.SRC_BF16)):
        ggml = ref.q8_0_from_hf(src, None, rdt)
        assert np.array_equal(_convert(src, None, dt, False), ggml)
        assert np.array_equal(_convert(src, None, dt, True), ref.q8_0_repack_rows(ggml, 24, inn // 32))
    assert np.array_equal(_convert(x, None, SRC_F32, True), ref.q8_0_quantize_rows(x))


@pytest.mark.parametrize("rows,blocks", [(7, 3), (16, 44), (5, 64)])
def test_q8_0_repack_rows_bit_exact(rows, blocks):
    rng = np.random.default_rng(rows + blocks)
    ggml = rng.integers(0, 256, rows * blocks * 34, dtype=np.uint8)
    dst = torch.zeros(ggml.size, dtype=torch.uint8, device="cuda")
    dispatch.q8_0_repack_rows(dst, dev(ggml), rows, blocks)
    assert np.array_equal(dst.cpu().numpy(), ref.q8_0_repack_rows(ggml, rows, blocks))


def test_converters_refuse_what_the_reference_refuses():
    codes = dev(np.zeros((64, 64), np.uint8))
    dst = torch.zeros(64 * 2 * 34, dtype=torch.uint8, device="cuda")
    with pytest.raises(capi.DsxError, match="without a scale"):
        dispatch.q8_0_weights_from_hf(dst, codes, None, SRC_F8E4M3, 64, 64)
    with pytest.raises(capi.DsxError, match="does not exactly tile"):
        dispatch.q8_0_weights_from_hf(dst, codes, dev(np.full((3, 2), 127, np.uint8)), SRC_F8E4M3, 64, 64)
    with pytest.raises(capi.DsxError, match="multiple of 32"):
        dispatch.q8_0_weights_from_hf(dst, codes, None, SRC_F32, 64, 48)
    with pytest.raises(capi.DsxError, match="source dtype"):
        dispatch.q8_0_weights_from_hf(dst, codes, None, 9, 64, 64)
    with pytest.raises(capi.DsxError, match="in place"):
        dispatch.q8_0_repack_rows(dst, dst, 64, 2)
    # empty matrices are a no-op, as every entry point treats them
    dispatch.q8_0_weights_from_hf(dst, codes, None, SRC_F32, 0, 64)
    dispatch.q8_0_repack_rows(dst, codes, 0, 2)

"""Pins the oracle's format code against the reference's golden vectors, its known-answer
tests, and independent closed forms (numpy float16, f64 dot products, brute force)."""
import json
import os

import numpy as np
import pytest

from oracle import ref

HERE = os.path.dirname(os.path.abspath(__file__))
E2M1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], np.float64)


def lcg_bytes(n, seed):
    s = seed
    out = np.empty(n, np.uint8)
    for i in range(n):
        s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = s >> 24
    return out


# ---- golden vector: llama.cpp's dequantize_row_mxfp4 -----------------------------------

def test_mxfp4_dequant_matches_llamacpp_golden_bits():
    g = json.load(open(os.path.join(HERE, "golden", "mxfp4_llamacpp_dequant.json")))
    c = g["construction"]
    blocks = lcg_bytes(c["n_blocks"] * 17, c["seed"])
    for i in range(c["n_blocks"]):
        blocks[i * 17] = c["e_base"] + i
    got = ref.mxfp4_dequant_ggml(blocks).view(np.uint32)
    want = np.array(g["f32_bits"], np.uint32)
    assert np.array_equal(got, want)


def test_mxfp4_v2_layout_equals_ggml_blocks():
    # v2 super-block = the same 8 ggml blocks rearranged: nibbles of block k at k*16,
    # scale at 128+k (kernels/src/mxfp4_tables.rs:10-36).
    rng = np.random.default_rng(1)
    ggml = rng.integers(0, 256, 16 * 17, dtype=np.uint8)
    for b in range(16):
        ggml[b * 17] = 100 + b
    v2 = np.empty(2 * 136, np.uint8)
    for s in range(2):
        for k in range(8):
            blk = ggml[(s * 8 + k) * 17:(s * 8 + k + 1) * 17]
            v2[s * 136 + k * 16: s * 136 + k * 16 + 16] = blk[1:]
            v2[s * 136 + 128 + k] = blk[0]
    a = ref.mxfp4_dequant_ggml(ggml)
    b = ref.mxfp4_dequant_v2(v2, 1, 512).reshape(-1)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_mxfp4_closed_form_e2m1_times_pow2():
    # kvalues * 2^(e-128) == E2M1 * 2^(e-127) for every code and every normal exponent.
    for e in (1, 2, 60, 119, 127, 128, 200, 250):
        blk = np.zeros(17, np.uint8)
        blk[0] = e
        blk[1:17] = np.arange(16, dtype=np.uint8) | (np.arange(16, dtype=np.uint8)[::-1] << 4)
        y = ref.mxfp4_dequant_ggml(blk).astype(np.float64)
        lo = E2M1[np.arange(16)] * 2.0 ** (e - 127)
        hi = E2M1[np.arange(16)[::-1]] * 2.0 ** (e - 127)
        want = np.concatenate([lo, hi]).astype(np.float32).astype(np.float64)
        assert np.array_equal(y, want), e


def test_e8m0_e4m3_known_answers():
    l = ref.lib()
    # core/src/hf_v41.rs:1335-1340
    assert l.dsx_ref_e8m0_to_f32(127) == 1.0
    assert l.dsx_ref_e8m0_to_f32(0) == 2.0 ** -127
    assert l.dsx_ref_e8m0_to_f32(254) == 2.0 ** 127
    assert np.isnan(l.dsx_ref_e8m0_to_f32(255))
    # core/src/hf_v41.rs:1323-1331
    assert l.dsx_ref_e4m3_to_f32(0x38) == 1.0
    assert l.dsx_ref_e4m3_to_f32(0x7E) == 448.0
    assert l.dsx_ref_e4m3_to_f32(0x08) == 2.0 ** -6
    assert l.dsx_ref_e4m3_to_f32(0x01) == 2.0 ** -9
    assert l.dsx_ref_e4m3_to_f32(0xB8) == -1.0
    assert np.float32(l.dsx_ref_e4m3_to_f32(0x80)).view(np.uint32) == 0x80000000
    assert np.isnan(l.dsx_ref_e4m3_to_f32(0x7F)) and np.isnan(l.dsx_ref_e4m3_to_f32(0xFF))
    # half-scale table: 2^(e-128) incl. the two denormal entries
    for e in range(0, 255):
        assert l.dsx_ref_e8m0_half_to_f32(e) == 2.0 ** (e - 128)


def test_e4m3_all_codes_against_ml_dtypes_free_formula():
    l = ref.lib()
    for b in range(256):
        if b & 0x7F == 0x7F:
            continue
        s, e, m = b >> 7, (b >> 3) & 0xF, b & 7
        want = (m * 2.0 ** -9) if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
        assert l.dsx_ref_e4m3_to_f32(b) == (-want if s else want)


def test_f16_conversions_against_numpy():
    l = ref.lib()
    bits = np.arange(0, 65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float32)
    for b in list(range(0, 65536, 7)) + [0x7C00, 0xFC00, 0x0001, 0x03FF, 0x0400, 0x8000]:
        got = l.dsx_ref_f16_to_f32(b)
        if np.isnan(vals[b]):
            assert np.isnan(got)
        else:
            assert got == vals[b]
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 4000),
        np.array([0.0, -0.0, 65504.0, 65520.0, 65519.99, 1e-8, 5.9604645e-08, 2.9802322e-08,
                  2.98023224e-08 * 1.0000001, np.inf, -np.inf, 6.1035156e-05], np.float32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    for x, w in zip(xs, want):
        assert l.dsx_ref_f32_to_f16(float(x)) == w, (x, hex(w))


def test_bf16_round_trip():
    l = ref.lib()
    for b in (0x3F80, 0xBF80, 0x0001, 0x7F7F, 0x4049):
        f = l.dsx_ref_bf16_to_f32(b)
        assert np.float32(f).view(np.uint32) == b << 16
        assert l.dsx_ref_f32_to_bf16(f) == b
    # ties to even
    assert l.dsx_ref_f32_to_bf16(float(np.uint32(0x3F808000).view(np.float32))) == 0x3F80
    assert l.dsx_ref_f32_to_bf16(float(np.uint32(0x3F818000).view(np.float32))) == 0x3F82


# ---- HF -> v2 repack -------------------------------------------------------------------

def test_repack_nibble_placement_known_answer():
    # core/src/hf_v41.rs:1360-1382: element k of block 0 has code k & 0xF; in the repacked
    # block, byte i holds element i (low nibble) and element 16+i (high nibble).
    packed = np.zeros((1, 128), np.uint8)
    packed[0, :16] = [((2 * i) & 0xF) | (((2 * i + 1) & 0xF) << 4) for i in range(16)]
    scale = np.full((1, 8), 0x7F, np.uint8)
    v2 = ref.mxfp4_repack_hf_to_v2(packed, scale)
    for i in range(16):
        assert v2[i] & 0xF == i & 0xF
        assert v2[i] >> 4 == (16 + i) & 0xF
    assert v2[128] == 0x7F


def test_repack_round_trip_and_values():
    rng = np.random.default_rng(3)
    out, nb = 5, 16
    packed = rng.integers(0, 256, (out, nb * 16), dtype=np.uint8)
    scale = rng.integers(100, 140, (out, nb), dtype=np.uint8)
    v2 = ref.mxfp4_repack_hf_to_v2(packed, scale)
    p2, s2 = ref.mxfp4_unpack_v2_to_hf(v2, out, nb)
    assert np.array_equal(p2, packed) and np.array_equal(s2, scale)
    # dequant(v2)[r, j] == E2M1[HF nibble j] * 2^(scale-127): element 2i is the LOW nibble
    # of HF byte i (docs/v41/ARCH_SPEC.md:176-177).
    y = ref.mxfp4_dequant_v2(v2, out, nb * 32).astype(np.float64)
    codes = np.empty((out, nb * 32), np.uint8)
    codes[:, 0::2] = packed & 0xF
    codes[:, 1::2] = packed >> 4
    want = E2M1[codes] * 2.0 ** (np.repeat(scale.astype(np.float64), 32, axis=1) - 127)
    assert np.array_equal(y, want)


# ---- E2M1 quantizer --------------------------------------------------------------------

def test_mxfp4_quantizer_is_nearest_grid_point_with_pow2_ceil_scale():
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((3, 512)) * 0.02).astype(np.float32)
    x[0, :32] = 0.0                       # all-zero block
    x[1, 0] = 6.0                         # amax exactly on a power of two boundary: 6/6 = 1
    x[1, 1:32] = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -0.75, -2.5] + [0.1] * 21
    v2 = ref.mxfp4_quantize_v2(x)
    y = ref.mxfp4_dequant_v2(v2, 3, 512).astype(np.float64)
    grid = np.array([0, .5, 1, 1.5, 2, 3, 4, 6])
    for r in range(3):
        for b in range(16):
            xb = x[r, b * 32:(b + 1) * 32].astype(np.float64)
            amax = max(np.abs(xb).max(), 6 * 2.0 ** -126)
            scale = 2.0 ** np.ceil(np.log2(amax / 6))
            e = v2[(r * 2 + b // 8) * 136 + 128 + b % 8]
            assert 2.0 ** (int(e) - 127) == scale
            q = np.clip(xb / scale, -6, 6)
            got = y[r, b * 32:(b + 1) * 32] / scale
            # nearest grid point; exact ties resolve to the even-mantissa code (0,1,2,4)
            d = np.abs(np.abs(q)[:, None] - grid[None, :])
            assert np.all(np.abs(np.abs(got) - np.abs(q)) <= d.min(axis=1) + 1e-12)
            assert np.all((got == 0) | (np.sign(got) == np.sign(q)))
    # tie cases of block (1, 0): scale 1 -> .25->0, .75->1, 1.25->1, 1.75->2, 2.5->2, 3.5->4, 5->4
    got = y[1, 1:11]
    assert list(got) == [0.0, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0, -0.0, -1.0, -2.0]


# ---- Q8_0 ------------------------------------------------------------------------------

def test_q8_0_block_known_answer():
    # core/src/hf_v41.rs:1343-1358
    x = np.zeros(32, np.float32)
    x[:4] = [254.0, -1.0, 0.75, -0.75]
    o = ref.q8_0_quantize_block(x)
    assert o[:2].view(np.float16)[0] == 2.0
    assert list(o[2:6].view(np.int8)) == [127, -1, 0, 0]   # -0.5 rounds away from zero
    assert not ref.q8_0_quantize_block(np.zeros(32, np.float32)).any()


def test_q8_0_rows_layout_and_dequant():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((4, 96)) * 0.02).astype(np.float32)
    rows = ref.q8_0_quantize_rows(x)
    assert rows.size == 4 * 3 * 34
    y = ref.q8_0_dequant_rows(rows, 4, 96)
    for r in range(4):
        row = rows[r * 102:(r + 1) * 102]
        d = row[:6].view(np.float16).astype(np.float32)            # [blocks x f16]
        q = row[6:].view(np.int8).reshape(3, 32).astype(np.float32)  # [blocks x 32 i8]
        for b in range(3):
            blk = ref.q8_0_quantize_block(x[r, b * 32:(b + 1) * 32])
            assert blk[:2].view(np.float16)[0] == row[b * 2:b * 2 + 2].view(np.float16)[0]
            assert np.array_equal(blk[2:], row[6 + b * 32: 6 + (b + 1) * 32])
        assert np.array_equal(y[r], (d[:, None] * q).reshape(-1))
        assert np.max(np.abs(y[r] - x[r])) <= np.abs(x[r]).max() / 127 * 0.51 + 1e-6


def _q8_0_blocks_numpy(f):
    """ggml Q8_0 blocks of f32 rows by numpy: d = amax/127 -> float16, q = round half away."""
    out, inn = f.shape
    blk = f.reshape(out, inn // 32, 32)
    amax = np.nanmax(np.abs(np.where(np.isnan(blk), 0, blk)), axis=2).astype(np.float32)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        idv = np.where(d == 0, np.float32(0), np.float32(1.0) / d).astype(np.float32)
        t = (blk * idv[:, :, None]).astype(np.float32)
    q = np.where(np.isnan(t), 0, np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)))
    q = np.clip(q, -128, 127).astype(np.int8)
    res = np.empty((out, inn // 32, 34), np.uint8)
    res[:, :, :2] = d.astype(np.float16).view(np.uint8).reshape(out, inn // 32, 2)
    res[:, :, 2:] = q.view(np.uint8)
    return res.reshape(-1)


def test_q8_0_from_fp8_checkpoint_against_torch_float8_decoders():
    # crates/v4flash-core/src/hf_v41.rs:728-805; the fp8 / e8m0 values come from torch's own
    # float8 dtypes (a third-party decoder), the scale grid is indexed here with numpy.repeat
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(21)
    out, inn, br, bc = 96, 192, 32, 64           # cells are not square: a transposed grid fails
    codes = rng.integers(0, 256, (out, inn), dtype=np.uint8)
    scale = rng.integers(110, 140, (out // br, inn // bc), dtype=np.uint8)
    scale[0, 0] = 255                            # a NaN scale: the whole cell quantizes to zero
    w = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    sc = torch.from_numpy(scale).view(torch.float8_e8m0fnu).float().numpy()
    with np.errstate(invalid="ignore"):
        f = (w * np.repeat(np.repeat(sc, br, axis=0), bc, axis=1)).astype(np.float32)
    got = ref.q8_0_from_hf(codes, scale, ref.SRC_F8E4M3)
    assert np.array_equal(got, _q8_0_blocks_numpy(f))
    assert not got.reshape(out, inn // 32, 34)[:br, : bc // 32].any()
    # a constant 1.0 (code 0x38) under distinct scales reads back as the scale of its cell
    ones = np.full((out, inn), 0x38, np.uint8)
    grid = (120 + np.arange(9, dtype=np.uint8)).reshape(3, 3)
    rows = ref.q8_0_repack_rows(ref.q8_0_from_hf(ones, grid, ref.SRC_F8E4M3), out, inn // 32)
    y = ref.q8_0_dequant_rows(rows, out, inn)
    want = np.repeat(np.repeat(np.exp2(grid.astype(np.float64) - 127), br, axis=0), bc, axis=1)
    assert np.allclose(y, want, rtol=2e-3, atol=0)


def test_q8_0_from_bf16_and_f32_checkpoint():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(22)
    x = (rng.standard_normal((8, 96)) * 0.02).astype(np.float32)
    bits = torch.from_numpy(x).bfloat16().view(torch.int16).numpy().view(np.uint16)
    xb = torch.from_numpy(x).bfloat16().float().numpy()
    assert np.array_equal(ref.q8_0_from_hf(bits, None, ref.SRC_BF16), _q8_0_blocks_numpy(xb))
    g = ref.q8_0_from_hf(x, None, ref.SRC_F32)
    assert np.array_equal(g, _q8_0_blocks_numpy(x))
    # split rows = the same blocks, scales first (crates/v4flash-kernels/src/weights.rs:225-240)
    assert np.array_equal(ref.q8_0_repack_rows(g, 8, 3), ref.q8_0_quantize_rows(x))
    b3 = g.reshape(8, 3, 34)
    manual = np.concatenate([b3[:, :, :2].reshape(8, -1), b3[:, :, 2:].reshape(8, -1)], axis=1)
    assert np.array_equal(ref.q8_0_repack_rows(g, 8, 3), manual.reshape(-1))


def test_q8_0_from_fp8_refuses_what_the_reference_refuses():
    codes = np.zeros((64, 64), np.uint8)
    with pytest.raises(ValueError):
        ref.q8_0_from_hf(codes, None, ref.SRC_F8E4M3)              # fp8 without scales
    with pytest.raises(ValueError):
        ref.q8_0_from_hf(codes, np.full((3, 2), 127, np.uint8), ref.SRC_F8E4M3)  # 64 % 3 != 0


def test_q8_0_activation_quantizer():
    rng = np.random.default_rng(6)
    x = rng.standard_normal(128).astype(np.float32)
    x[32:64] = 0
    x[64] = 0.5 * 127 / 127  # exercise half-way rounding via lrintf (ties to even)
    xq, xs = ref.q8_0_quantize_act(x)
    for b in range(4):
        xb = x[b * 32:(b + 1) * 32]
        d = np.float32(np.abs(xb).max()) / np.float32(127.0)
        assert xs[b] == d
        if d == 0:
            assert not xq[b * 32:(b + 1) * 32].any()
            continue
        idv = np.float32(1.0) / d
        want = np.clip(np.rint(xb * idv), -128, 127).astype(np.int8)  # rint = half to even
        assert np.array_equal(xq[b * 32:(b + 1) * 32], want)


def test_q8_0_dot_equals_f64_dequant_dot():
    rng = np.random.default_rng(7)
    for cols in (2048, 1408, 64):
        w = (rng.standard_normal((1, cols)) * 0.02).astype(np.float32)
        x = rng.standard_normal(cols).astype(np.float32)
        rows = ref.q8_0_quantize_rows(w)
        xq, xs = ref.q8_0_quantize_act(x)
        got = ref.dot_q8_0(rows, xq, xs)
        wd = ref.q8_0_dequant_rows(rows, 1, cols)[0].astype(np.float64)
        xd = xq.astype(np.float64) * np.repeat(xs.astype(np.float64), 32)
        want = float(wd @ xd)
        assert abs(got - want) <= 1e-5 * np.abs(wd * xd).sum()


# ---- Q8_K ------------------------------------------------------------------------------

def q8k_numpy(x):
    """Independent restatement in numpy of the rule in kernels/tests/q8_k_quantize.rs."""
    out = []
    for xb in x.reshape(-1, 256):
        i = int(np.argmax(np.abs(xb)))          # first maximum
        if xb[i] == 0:
            out.append((np.float32(0), np.zeros(256, np.int8)))
            continue
        iscale = np.float32(-127.0) / xb[i]
        q = np.clip(np.rint(iscale * xb), -128, 127).astype(np.int8)
        out.append((np.float32(1.0) / iscale, q))
    return out


def test_q8k_quantize_bit_exact_and_invariants():
    rng = np.random.default_rng(8)
    x = rng.standard_normal(256 * 6).astype(np.float32)
    x[256:512] = 0                                   # zero block
    x[512:768] = -np.abs(x[512:768])                 # negative maximum
    x[768] = 3.0; x[769] = -3.0                      # tie in |x|: the first one wins
    x[768 + 2: 1024] *= 0.1
    blocks = ref.q8k_quantize(x)
    assert blocks.size == 6 * 292
    for b, (d, q) in enumerate(q8k_numpy(x)):
        blk = blocks[b * 292:(b + 1) * 292]
        assert blk[:4].view(np.float32)[0] == d
        qs = blk[4:260].view(np.int8)
        assert np.array_equal(qs, q)
        bs = blk[260:].view(np.int16)
        assert np.array_equal(bs, q.reshape(16, 16).astype(np.int32).sum(axis=1))
        if d != 0:
            assert qs[int(np.argmax(np.abs(x[b * 256:(b + 1) * 256])))] == -127
    assert not blocks[292:584].any()
    assert blocks[3 * 292 + 4: 3 * 292 + 6].view(np.int8).tolist() == [-127, 127]


def test_dot_mxfp4_q8k_equals_f64_dequant_dot():
    # property from external/ds4-dump/quants_selftest.c:120-171 (1e-4 relative)
    c = dict(seed=0x53)
    n = 4 * 256
    ggml = lcg_bytes(n // 32 * 17, c["seed"])
    for i in range(n // 32):
        ggml[i * 17] = 118 + i
    s = c["seed"] ^ 0xabcdef01
    x = np.empty(n, np.float32)
    for i in range(n):
        s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
        x[i] = (np.float32(s >> 24) - np.float32(127.5)) / np.float32(64.0)
    v2 = np.empty(4 * 136, np.uint8)
    for sb in range(4):
        for k in range(8):
            blk = ggml[(sb * 8 + k) * 17:(sb * 8 + k + 1) * 17]
            v2[sb * 136 + k * 16: sb * 136 + (k + 1) * 16] = blk[1:]
            v2[sb * 136 + 128 + k] = blk[0]
    xq = ref.q8k_quantize(x)
    got = ref.dot_mxfp4_q8k(v2, xq)
    want = float(ref.mxfp4_dequant_ggml(ggml).astype(np.float64) @ ref.q8k_dequant(xq).astype(np.float64))
    assert abs(got - want) / max(abs(want), 1e-6) < 1e-4


def test_dot_mxfp4_q8k_brute_force_tiny():
    # one-hot activations read back single dequantized weights exactly
    rng = np.random.default_rng(9)
    v2 = rng.integers(0, 256, 136, dtype=np.uint8)
    v2[128:] = rng.integers(110, 130, 8)
    w = ref.mxfp4_dequant_v2(v2, 1, 256)[0]
    for j in (0, 15, 16, 31, 32, 100, 255):
        xq = np.zeros(292, np.uint8)
        xq[:4] = np.array([1.0], np.float32).view(np.uint8)
        xq[4 + j] = 1
        assert ref.dot_mxfp4_q8k(v2, xq) == w[j]
    # transposed-operand guard: a ramp activation distinguishes element order
    xq = np.zeros(292, np.uint8)
    xq[:4] = np.array([0.5], np.float32).view(np.uint8)
    xq[4:260] = (np.arange(256) % 127).astype(np.int8).view(np.uint8)
    want = 0.5 * float(w.astype(np.float64) @ (np.arange(256) % 127))
    assert abs(ref.dot_mxfp4_q8k(v2, xq) - want) <= 1e-6 * abs(want) + 1e-30


# ---- swiglu / rmsnorm ------------------------------------------------------------------

def test_swiglu_closed_form_and_clamp_edges():
    f = ref.swiglu
    sig = lambda g: 1.0 / (1.0 + np.exp(-g))
    assert abs(f(1.5, -2.0, 0.0, 0.7) - 1.5 * sig(1.5) * -2.0 * 0.7) < 1e-6
    assert abs(f(15.0, 3.0, 10.0, 1.0) - 10 * sig(10.0) * 3.0) < 1e-5       # gate clamped above
    assert abs(f(-15.0, 3.0, 10.0, 1.0) - (-15 * sig(-15.0) * 3.0)) < 1e-9  # not below
    assert abs(f(1.0, 30.0, 10.0, 1.0) - sig(1.0) * 10.0) < 1e-5
    assert abs(f(1.0, -30.0, 10.0, 1.0) + sig(1.0) * 10.0) < 1e-5
    assert abs(f(15.0, 30.0, 1e-6, 1.0) - 15 * sig(15.0) * 30) < 1e-3       # clamp disabled
    assert f(10.0, 10.0, 10.0, 1.0) == f(10.0, 10.0, 0.0, 1.0)


def test_rms_norm_closed_form():
    rng = np.random.default_rng(10)
    x = rng.standard_normal((3, 7168)).astype(np.float32)
    w = (1 + 0.02 * rng.standard_normal(7168)).astype(np.float32)
    got = ref.rms_norm(x, w, 1e-6)
    xd = x.astype(np.float64)
    want = xd / np.sqrt((xd ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
    assert np.max(np.abs(got - want)) < 2e-6 * np.abs(want).max()


def test_wi_upper_bound_known_answers_and_brute_force():
    # kernels/src/het/dispatch.rs:721-749
    assert ref.wi_upper_bound(12, 384, 32, 10 ** 6) == 12
    assert ref.wi_upper_bound(3072, 384, 32, 10 ** 6) == 480
    rng = np.random.default_rng(11)
    for _ in range(200):
        m, g, c = int(rng.integers(1, 200)), int(rng.integers(1, 40)), int(rng.integers(1, 33))
        sizes = np.bincount(rng.integers(0, g, m), minlength=g)
        exact = int(sum(-(-s // c) for s in sizes))
        assert ref.wi_upper_bound(m, g, c, 10 ** 6) >= exact

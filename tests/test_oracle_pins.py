"""Pins the CPU oracle against what the reference's own tests hold for this path and against what
the mathematics fixes, without running the reference.

- REF_HASHES (src/ggml.rs:1547-1577): FNV-1a-64 of gguf-py's dequantization of the seeded fixtures.
- f16 / bf16 conversions: exhaustive against numpy / torch.
- e4m3: all 256 bytes against torch.float8_e4m3fn and the closed form (src/ggml.rs:1505-1523).
- quantize_act: the scalar definition of src/quant.rs:633-658 including its special cases.
- decode_i8: the invariant of src/ggml.rs:1663-1681.
"""
import json
import os

import numpy as np
import pytest
import torch

# (type id, hash): the reference's golden table (src/ggml.rs:1547-1577), kept as a fixture
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_hashes.json")) as _f:
    _GOLDEN = json.load(_f)
REF_HASHES = {name: (e["ggml_type"], int(e["fnv1a64"], 16)) for name, e in _GOLDEN["hashes"].items()}
FIXTURE_ELEMS = _GOLDEN["elements"]


def fixture_blocks(oxref, kind):
    raw, _ = oxref.random_blocks(kind, FIXTURE_ELEMS // oxref.block_size(kind), 1000 + kind)
    return raw


@pytest.mark.parametrize("name", sorted(REF_HASHES))
def test_dequantization_matches_ggml_hashes(oxref, name):
    kind, want = REF_HASHES[name]
    y = oxref.dequantize_row(kind, fixture_blocks(oxref, kind), FIXTURE_ELEMS)
    assert oxref.fnv1a_f32(y) == want, f"{name}: dequantized fixture differs from ggml"


def test_fnv_known_answer(oxref):
    # FNV-1a-64 of the empty input is the offset basis; of one zero byte quadruple a fixed value.
    assert oxref.fnv1a_f32(np.zeros(0, np.float32)) == 0xcbf29ce484222325
    h = 0xcbf29ce484222325
    for b in np.float32(1.5).tobytes():
        h = ((h ^ b) * 0x100000001b3) % (1 << 64)
    assert oxref.fnv1a_f32(np.array([1.5], np.float32)) == h


def test_lcg_known_answers(oxref):
    s, out = 7, []
    for _ in range(4):
        s = (s * 6364136223846793005 + 1442695040888963407) % (1 << 64)
        out.append(s >> 33)
    got, end = oxref.lcg_stream(7, 4)
    assert list(got) == out and end == s


def test_f16_to_f32_exhaustive(oxref):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oxref.lib.oxref_f16_to_f32(int(v)) for v in h], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


def test_f32_to_f16_rne(oxref):
    rng = np.random.default_rng(1)
    # every f16 value, the midpoints between neighbours, values just off them, and random bits
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = (h[:-1] + h[1:]) / 2
    vals = np.concatenate([h, mids, np.nextafter(mids.astype(np.float32), np.float32(np.inf)).astype(np.float64),
                           np.nextafter(mids.astype(np.float32), np.float32(-np.inf)).astype(np.float64),
                           [65504.0, 65519.9, 65520.0, 1e9, 2.0 ** -25, 2.0 ** -24, 1.0000001 * 2.0 ** -25, 0.0]])
    vals = np.concatenate([vals, -vals]).astype(np.float32)
    rnd = rng.integers(0, 1 << 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    rnd = rnd[np.isfinite(rnd)]
    for x in (vals, rnd):
        with np.errstate(over="ignore"):
            want = x.astype(np.float16).view(np.uint16)
        got = np.array([oxref.lib.oxref_f32_to_f16(float(v)) for v in x], np.uint16)
        assert np.array_equal(got, want)


def test_f32_to_bf16_rne(oxref):
    rng = np.random.default_rng(2)
    x = rng.integers(0, 1 << 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    x = x[np.isfinite(x)]
    x = np.concatenate([x, np.array([1.0, 1.00390625, 1.005859375, 1.001953125, 3.3895314e38, -0.0], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([oxref.lib.oxref_f32_to_bf16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)
    back = np.array([oxref.lib.oxref_bf16_to_f32(int(v)) for v in got[:1000]], np.float32)
    assert np.array_equal(back.view(np.uint32), (got[:1000].astype(np.uint32) << 16))


def test_e4m3_all_bytes(oxref):
    b = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(b).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = np.array([oxref.e4m3_to_f32(v) for v in b], np.float32)
    nan = np.isnan(want)
    assert list(np.nonzero(nan)[0]) == [0x7F, 0xFF]
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert got[0x7E] == 448.0 and got[0x01] == 2.0 ** -9 and got[0x08] == 2.0 ** -6


def test_e4m3_scaled_matches_the_table(oxref):
    # src/ggml.rs:1505-1523: the bit-built conversion times s equals the table value times s
    bytes_ = np.concatenate([np.arange(256), np.arange(255, -1, -1)]).astype(np.uint8)
    table = np.array([oxref.e4m3_to_f32(v) for v in range(256)], np.float32)
    for s in (1.0, 0.003741, -2.5):
        for n in (0, 1, 7, 16, 33, 128, 300, 512):
            got = oxref.e4m3_scaled(bytes_[:n], s)
            want = table[bytes_[:n]] * np.float32(s)
            nan = np.isnan(want)
            assert np.array_equal(np.isnan(got), nan)
            assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


def test_fp8_block_scale_indexing(oxref):
    # scale of weight (r, c) is s[(r / rows) * ceil(n_in / cols) + c / cols] (src/ggml.rs:250-256)
    n_out, n_in = 256, 320  # 3 column blocks, the last partial
    data = np.full((n_out, n_in), 0x38, np.uint8)  # 1.0
    scales = np.arange(1, 2 * 3 + 1, dtype=np.float32)
    w = oxref.fp8_dequant_rows(data, scales, n_out, n_in)
    for r, c in [(0, 0), (127, 127), (127, 128), (128, 0), (255, 319), (130, 256)]:
        assert w[r, c] == scales[(r // 128) * 3 + c // 128]


def test_activation_quantization_matches_scalar(oxref):
    # src/quant.rs:633-658
    t, n = 5, 4 * 32
    s, xs = 7, []
    for _ in range(t * n):
        s = (s * 6364136223846793005 + 1442695040888963407) % (1 << 64)
        xs.append(np.float32((s >> 33) % 20001) / np.float32(1000.0) - np.float32(10.0))
    x = np.array(xs, np.float32)
    x[32:64] = 0.0
    x[2 * 32 + 3] = 1e-30
    for tt in (1, t):
        q, scales, sums, fsums, hsums = oxref.quantize_act(x[: tt * n], tt, n)
        q, scales, sums, fsums, hsums = (a.reshape(-1) for a in (q, scales, sums, fsums, hsums))
        for bi in range(tt * n // 32):
            blk = x[bi * 32:(bi + 1) * 32]
            amax = np.float32(0)
            for v in blk:
                amax = max(amax, np.float32(abs(v)))
            inv = np.float32(127.0) / amax if amax > 0 else np.float32(0)
            p = blk * inv
            qq = (np.sign(p) * np.floor(np.abs(p) + np.float32(0.5))).astype(np.int8)  # half away from zero
            assert np.array_equal(q[bi * 32:(bi + 1) * 32], qq), bi
            assert scales[bi].view(np.uint32) == (amax / np.float32(127.0)).view(np.uint32)
            assert sums[bi] == int(qq.astype(np.int32).sum())
            acc = np.float32(0)
            for v in blk:
                acc = np.float32(acc + v)
            assert fsums[bi].view(np.uint32) == acc.view(np.uint32)
            acc = np.float32(0)
            for v in blk[16:]:
                acc = np.float32(acc + v)
            assert hsums[2 * bi + 1].view(np.uint32) == acc.view(np.uint32)
        assert np.all(q[32:64] == 0) and scales[1] == 0.0


@pytest.mark.parametrize("name", [k for k in sorted(REF_HASHES) if k not in ("F32", "F16", "BF16")])
def test_int8_decoding_matches_dequantization(oxref, name):
    # src/ggml.rs:1663-1681
    kind, _ = REF_HASHES[name]
    raw = fixture_blocks(oxref, kind)
    want = oxref.dequantize_row(kind, raw, FIXTURE_ELEMS)
    bs, ts = oxref.block_size(kind), oxref.type_size(kind)
    for bi in range(FIXTURE_ELEMS // bs):
        q, s, m, has_min = oxref.decode_i8(kind, raw[bi * ts:(bi + 1) * ts])
        if not has_min:
            m[:] = 0
        v = np.repeat(s, 16) * q.astype(np.float32) + np.repeat(m, 16)
        w = want[bi * bs:(bi + 1) * bs]
        assert np.all(np.abs(v - w) <= 1e-6 * np.maximum(np.abs(w), 1e-3)), (name, bi)


def test_type_geometry(oxref):
    # src/ggml.rs:1683-1690 and the row sizes of the benchmark shapes
    assert oxref.row_bytes(12, 5120) == 20 * 144
    assert oxref.row_bytes(8, 4096) == 4352 and oxref.row_bytes(12, 4096) == 2304 and oxref.row_bytes(14, 4096) == 3360
    assert oxref.block_size(15) == 0  # Q8_K is not a weight format


def test_nvfp4_against_the_format_definitions(oxref):
    """NVFP4 (src/ggml.rs:79-83, :477-490, :936-947), which has no entry in the reference's hash table: every (scale byte,
    code) pair against what the formats themselves define. The scale is an unsigned E4M3 value, halved (torch's
    float8_e4m3fn decodes the byte's low seven bits; 0 and 0x7f give 0, the top bit is ignored); the codes are E2M1 values
    (sign, two exponent bits, one mantissa bit: 0, 0.5, 1, 1.5, 2, 3, 4, 6), stored doubled. A block of 64 is four
    sub-blocks of 16: scale byte s, then 8 bytes whose byte j holds elements j (low nibble) and j + 8 (high)."""
    e4m3 = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()

    def e2m1(code):
        sign, e, m = -1.0 if code & 8 else 1.0, (code >> 1) & 3, code & 1
        return sign * (m * 0.5 if e == 0 else (1 + m / 2) * 2.0 ** (e - 1))
    for sc in range(256):
        low7 = sc & 0x7F
        want_scale = 0.0 if sc in (0, 0x7F) else (480.0 if sc == 0xFF else float(e4m3[low7])) * 0.5  # 0xff: e = 15, m = 7 read as a number, 1.875 * 2^8
        assert oxref.ue4m3_half(sc) == want_scale, sc
        # one block: sub-block 1 carries this scale, its 16 elements walk the 16 codes in an order that tells low from
        # high nibbles and byte j from byte j + 1; the other sub-blocks carry other scales and codes
        blk = np.zeros(36, np.uint8)
        blk[0:4] = [0x38, sc, 0x30, 0x41]
        codes = [(5 * i + 3) % 16 for i in range(16)]
        for j in range(8):
            blk[4 + 8 + j] = codes[j] | (codes[j + 8] << 4)
            blk[4 + j] = 0x21
            blk[4 + 16 + j] = 0x9C
            blk[4 + 24 + j] = 0x5F
        y = oxref.dequantize_row(oxref.NVFP4, blk, 64)
        want = np.array([np.float32(want_scale) * np.float32(2 * e2m1(c) + 0.0) for c in codes], np.float32)  # (the table is integers: code 8 is +0)
        assert np.array_equal(y[16:32].view(np.uint32), want.view(np.uint32)), sc
        assert y[0] == np.float32(0.5) * np.float32(2 * e2m1(1)) and y[8] == np.float32(0.5) * np.float32(2 * e2m1(2))
        assert y[32] == np.float32(0.25) * np.float32(2 * e2m1(0xC)) and y[40] == np.float32(0.25) * np.float32(2 * e2m1(9))
    assert oxref.block_size(oxref.NVFP4) == 64 and oxref.type_size(oxref.NVFP4) == 36 and oxref.row_bytes(oxref.NVFP4, 128) == 72
    # the matrix's scale on top of the decoded values: one more f32 multiply (src/ggml.rs:420-432), here per 2 x 64 block
    from oxinfer_amd import synth
    raw, _ = synth.gguf_nvfp4(4, 128, 3)
    s = np.array([[2.0, 0.5], [3.0, 0.75]], np.float32)
    got = oxref.gguf_dequant_rows_scaled(oxref.NVFP4, raw, s, 4, 128, 2, 64)
    base = oxref.dequantize_rows(oxref.NVFP4, raw, 4, 128)
    assert np.array_equal(got, base * np.repeat(np.repeat(s, 2, axis=0), 64, axis=1))
    assert np.array_equal(oxref.gguf_dequant_rows_scaled(oxref.NVFP4, raw, None, 4, 128), base)
    # the matmul is the f32 product of those rows (float-stored: the f32 path at every token count)
    x = synth.activations(3, 128, 4)
    y = oxref.gemm_quant(oxref.NVFP4, raw, s, None, 4, 128, x, 3, brows=2, bcols=64)
    assert np.abs(y - x.astype(np.float64) @ got.astype(np.float64).T).max() < 1e-4 * np.abs(y).max()

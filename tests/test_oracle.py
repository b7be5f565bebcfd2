"""Pins oracle/oracle_ops.c — the CPU restatement used as the checker — against (a) the reference's own compiled code
in oracle/_ref (libggml-base quantizers, the ggml CPU backend run on one-op graphs) and (b) closed forms that do not
share its structure (float64 numpy GEMM / softmax / layer norm, exhaustive bit patterns).  A dropped term, a wrong
nibble order, a transposed operand or a wrong rounding mode fails at least one of these."""
from __future__ import annotations

import numpy as np
import pytest

RNG = np.random.default_rng(20251125)


def rnd(shape, scale=1.0, offset=0.0):
    return (RNG.normal(size=shape) * scale + offset).astype(np.float32)


# ------------------------------------------------------------------------------------------------------------------
# f16 conversions
# ------------------------------------------------------------------------------------------------------------------

def test_f16_to_f32_all_bit_patterns(oracle, ref):
    h = np.arange(65536, dtype=np.uint16)
    mine, theirs, np16 = oracle.f16_bits_to_f32(h), ref.fp16_to_fp32(h), h.view(np.float16).astype(np.float32)
    assert np.array_equal(mine.view(np.uint32)[~np.isnan(np16)], np16.view(np.uint32)[~np.isnan(np16)])
    assert np.array_equal(np.isnan(mine), np.isnan(np16))
    assert np.array_equal(mine.view(np.uint32)[~np.isnan(theirs)], theirs.view(np.uint32)[~np.isnan(theirs)])


def test_f32_to_f16_round_to_nearest_even(oracle, ref):
    # every f16 value, both neighbours' midpoints (ties) and just-off-midpoints, plus random floats over the whole range
    h = np.arange(0, 0x7C00, dtype=np.uint16)
    v = h.view(np.float16).astype(np.float64)
    nxt = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = (v + nxt) / 2
    xs = np.concatenate([v, mid, np.nextafter(mid.astype(np.float32), np.float32(np.inf)), np.nextafter(mid.astype(np.float32), np.float32(-np.inf)),
                         RNG.normal(size=20000) * 10.0 ** RNG.integers(-9, 6, size=20000), [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e30, 5.96e-8, 2.98e-8, 2.99e-8]])
    xs = np.concatenate([xs, -xs]).astype(np.float32)
    mine = oracle.f32_to_f16_bits(xs)
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)            # numpy rounds to nearest even
    assert np.array_equal(mine, want)
    assert np.array_equal(mine, ref.fp32_to_fp16(xs))


# ------------------------------------------------------------------------------------------------------------------
# block formats
# ------------------------------------------------------------------------------------------------------------------

def test_dequantize_q5_0_every_nibble_and_high_bit(oracle, ref):
    # closed form: w = d * ((nibble | highbit << 4) - 16); element j < 16 is the low nibble of byte j, j >= 16 the high nibble of byte j - 16
    blocks = np.zeros((256, 22), dtype=np.uint8)
    for b in range(256):
        blocks[b, 0:2] = np.frombuffer(np.float16(0.5 + b / 64).tobytes(), dtype=np.uint8)
        blocks[b, 2:6] = np.frombuffer(np.uint32((b * 0x01010101) ^ (0xA5A5A5A5 if b % 2 else 0)).tobytes(), dtype=np.uint8)
        blocks[b, 6:22] = (np.arange(16) * 17 + b) % 256
    got = oracle.dequantize(oracle.Q5_0, blocks, 32)
    want = np.empty((256, 32), dtype=np.float32)
    for b in range(256):
        d = np.float32(np.frombuffer(blocks[b, 0:2].tobytes(), dtype=np.float16)[0])
        qh = int(np.frombuffer(blocks[b, 2:6].tobytes(), dtype=np.uint32)[0])
        for j in range(32):
            byte = int(blocks[b, 6 + j % 16])
            nib = (byte & 0xF) if j < 16 else (byte >> 4)
            want[b, j] = np.float32(((nib | (((qh >> j) & 1) << 4)) - 16)) * d
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got.view(np.uint32), ref.dequantize_row(ref.Q5_0, blocks, 32).view(np.uint32))


def test_dequantize_q8_0_all_quants(oracle, ref):
    blocks = np.zeros((8, 34), dtype=np.uint8)
    for b in range(8):
        blocks[b, 0:2] = np.frombuffer(np.float16(0.013 * (b + 1)).tobytes(), dtype=np.uint8)
        blocks[b, 2:34] = np.arange(32 * b, 32 * b + 32) % 256          # every int8 value appears
    got = oracle.dequantize(oracle.Q8_0, blocks, 32)
    d = np.array([np.float32(np.float16(0.013 * (b + 1))) for b in range(8)], dtype=np.float32)
    want = blocks[:, 2:].view(np.int8).astype(np.float32) * d[:, None]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got.view(np.uint32), ref.dequantize_row(ref.Q8_0, blocks, 32).view(np.uint32))


@pytest.mark.parametrize("wtype", ["Q5_0", "Q8_0"])
def test_model_file_quantizers_match_reference_bytes(oracle, ref, wtype):
    t = getattr(oracle, wtype)
    x = rnd((64, 256), 0.02)
    x[0, :32] = 0.0                      # all-zero block: d = 0, id = 0
    x[1, 5] = 3.0                        # outlier
    x[2, :32] = -np.abs(x[2, :32])       # negative extreme: q5_0 takes the signed value of largest magnitude
    x[3, 0:32] = np.linspace(-1, 1, 32)  # exact .5 steps after scaling exercise the rounding rule
    assert np.array_equal(oracle.quantize(t, x), ref.quantize_chunk(t, x).reshape(64, -1))
    # closed-form property: |dequant - x| <= d/2 (q8_0) resp. d (q5_0: 32 levels for a range of 31 steps), plus the f16 rounding of d
    deq = oracle.dequantize(t, oracle.quantize(t, x), 256)
    blk_amax = np.abs(x).reshape(64, 8, 32).max(-1, keepdims=True)
    step = blk_amax / (127 if t == oracle.Q8_0 else 16)
    assert np.all(np.abs(deq.reshape(64, 8, 32) - x.reshape(64, 8, 32)) <= step * (0.57 if t == oracle.Q8_0 else 1.02) + 1e-12)


def test_activation_quantizer_matches_cpu_backend(oracle, ref):
    x = rnd((16, 128), 1.7)
    x[0, :32] = 0.0
    x[1, :32] = np.arange(32) - 15.5     # scaled values land on .5: half-to-even vs half-away differ here
    mine = oracle.quantize(oracle.Q8_0, x, act=True)
    assert np.array_equal(mine, ref.quantize_row_q8_0_cpu(x))


# ------------------------------------------------------------------------------------------------------------------
# MUL_MAT
# ------------------------------------------------------------------------------------------------------------------

def _weights(oracle, wtype, m, k):
    w = rnd((m, k), 0.02)
    if wtype in (oracle.Q5_0, oracle.Q8_0):
        blocks = oracle.quantize(wtype, w)
        return blocks, oracle.dequantize(wtype, blocks, k)
    if wtype == oracle.F16:
        bits = oracle.f32_to_f16_bits(w)
        return bits, oracle.f16_bits_to_f32(bits)
    return w, w


@pytest.mark.parametrize("wtype", ["Q5_0", "Q8_0", "F16", "F32"])
@pytest.mark.parametrize("n", [1, 5, 33])
def test_mul_mat_against_cpu_backend_and_float64(oracle, ref, wtype, n):
    t = getattr(oracle, wtype)
    m, k = 48, 256
    wdata, wdeq = _weights(oracle, t, m, k)
    x = rnd((n, k))
    got = oracle.mul_mat(t, wdata, x)
    with ref.Graph() as g:
        tw = g.tensor(t, wdata, ne=[k, m])
        tx = g.tensor(ref.F32, x)
        want = g.run(g.op("ggml_mul_mat", tw, tx), out_shape=(n, m))
    assert oracle.nmse(got, want) < 1e-12, "restatement differs from the reference's CPU MUL_MAT"
    # float64 GEMM of the dequantized weights: differs only by the activation rounding the reference applies
    exact = x.astype(np.float64) @ wdeq.astype(np.float64).T
    bound = {oracle.Q5_0: 2e-4, oracle.Q8_0: 2e-4, oracle.F16: 1e-6, oracle.F32: 1e-12}[t]
    assert oracle.nmse(got, exact) < bound
    if t in (oracle.Q5_0, oracle.Q8_0):
        assert oracle.nmse(got, exact) > 1e-7, "the Q8_0 rounding of the activations is missing"
    # transposed-operand guard: the result is [n, m], not [m, n]
    assert got.shape == (n, m)


def test_mul_mat_one_hot_returns_weight_row(oracle):
    # x = e_j * 127 quantizes exactly (d = 1, q = 127): the product is 127 * w[:, j], tying MUL_MAT to dequantization
    m, k = 16, 64
    blocks, wdeq = _weights(oracle, oracle.Q5_0, m, k)
    for j in (0, 15, 16, 31, 32, 63):
        x = np.zeros((1, k), dtype=np.float32)
        x[0, j] = 127.0
        got = oracle.mul_mat(oracle.Q5_0, blocks, x)[0]
        assert np.allclose(got, 127.0 * wdeq[:, j], rtol=1e-6, atol=0)


def test_mul_mat_f16_f16_conv_operands(oracle, ref):
    a = oracle.f32_to_f16_bits(rnd((40, 96)))
    b = oracle.f32_to_f16_bits(rnd((24, 96), 0.02))
    got = oracle.mul_mat_f16_f16(a, b)
    with ref.Graph() as g:
        want = g.run(g.op("ggml_mul_mat", g.tensor(ref.F16, a), g.tensor(ref.F16, b)), out_shape=(24, 40))
    assert oracle.nmse(got, want) < 1e-12
    exact = oracle.f16_bits_to_f32(b).astype(np.float64) @ oracle.f16_bits_to_f32(a).astype(np.float64).T
    assert oracle.nmse(got, exact) < 1e-10


# ------------------------------------------------------------------------------------------------------------------
# FLASH_ATTN_EXT
# ------------------------------------------------------------------------------------------------------------------

def _exact_attention(oracle, q, kb, vb, mask, scale):
    qf = oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(q)).astype(np.float64)
    kf, vf = oracle.f16_bits_to_f32(kb).astype(np.float64), oracle.f16_bits_to_f32(vb).astype(np.float64)
    s = np.einsum("hnd,hkd->hnk", qf, kf) * scale
    if mask is not None:
        s = s + oracle.f16_bits_to_f32(mask).astype(np.float64)[None, :, :]
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    return np.einsum("hnk,hkd->nhd", p, vf)


@pytest.mark.parametrize("case", ["peaked", "flat_mean_dominated_padded", "masked"])
def test_flash_attn_against_cpu_backend_and_float64(oracle, ref, case):
    H, N, KV, D = 2, 7, 200, 64
    q = rnd((H, N, D), 1.0 if case != "flat_mean_dominated_padded" else 0.05)
    k, v = rnd((H, KV, D)), rnd((H, KV, D), 0.3, 1.0 if case == "flat_mean_dominated_padded" else 0.0)
    if case == "flat_mean_dominated_padded":     # whisper's kv_pad: trailing keys never written, all zero
        k[:, 180:] = 0.0
        v[:, 180:] = 0.0
    kb, vb = oracle.f32_to_f16_bits(k), oracle.f32_to_f16_bits(v)
    mask = None
    if case == "masked":
        m = np.full((64, KV), -np.inf, dtype=np.float32)      # rows padded to 64 like GGML_KQ_MASK_PAD
        for r in range(N):
            m[r, : KV // 2] = 0.0
            m[r, KV // 2 + r :: N] = 0.0
        mask = oracle.f32_to_f16_bits(m)
    got = oracle.flash_attn_ext(q, kb, vb, None if mask is None else mask[:N], 0.125)
    with ref.Graph() as g:
        tq, tk, tv = g.tensor(ref.F32, q), g.tensor(ref.F16, kb), g.tensor(ref.F16, vb)
        tm = g.tensor(ref.F16, mask) if mask is not None else None
        want = g.run(g.op("ggml_flash_attn_ext", tq, tk, tv, tm, 0.125, 0.0, 0.0), out_shape=(N, H, D))
    assert oracle.nmse(got, want) < 1e-7, "restatement differs from the reference's CPU FLASH_ATTN_EXT"  # f16 roundings flip where the SIMD dot product differs in the last bit
    exact = _exact_attention(oracle, q, kb, vb, None if mask is None else mask[:N], 0.125)
    assert oracle.nmse(got, exact) < 2e-3          # the f16 accumulator costs up to ~1e-3 on flat, mean-dominated data
    # invariant: identical V rows come back unchanged (softmax weights sum to one)
    vconst = np.broadcast_to(rnd((1, 1, D)), (H, KV, D)).copy()
    out = oracle.flash_attn_ext(q, kb, oracle.f32_to_f16_bits(vconst), None, 0.125)
    assert np.allclose(out, oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(vconst[:, :1].transpose(1, 0, 2))), rtol=2e-2)


# ------------------------------------------------------------------------------------------------------------------
# row / elementwise ops
# ------------------------------------------------------------------------------------------------------------------

def test_norm(oracle, ref):
    x = rnd((9, 320), 2.0, 0.7)
    got = oracle.norm(x, 1e-5)
    with ref.Graph() as g:
        want = g.run(g.op("ggml_norm", g.tensor(ref.F32, x), 1e-5), out_shape=x.shape)
    assert oracle.nmse(got, want) < 1e-12
    x64 = x.astype(np.float64)
    exact = (x64 - x64.mean(-1, keepdims=True)) / np.sqrt(x64.var(-1, keepdims=True) + 1e-5)
    assert oracle.nmse(got, exact) < 1e-12
    assert np.allclose(got.mean(-1), 0, atol=1e-6) and np.allclose(got.var(-1), 1, atol=1e-4)


def test_gelu(oracle, ref):
    x = np.concatenate([rnd((4000,), 3.0), np.array([-11, -10, -9.99, 0, 9.99, 10, 11, 1e-4], dtype=np.float32)])
    got = oracle.gelu(x)
    with ref.Graph() as g:
        want = g.run(g.op("ggml_gelu", g.tensor(ref.F32, x)), out_shape=x.shape)
    assert np.array_equal(got, want), "GELU through the f16 table is reproduced bit for bit"
    # ... for every f16 argument the table can be asked about
    allx = oracle.f16_bits_to_f32(np.arange(65536, dtype=np.uint16))
    allx = allx[np.isfinite(allx)]
    with ref.Graph() as g:
        want_all = g.run(g.op("ggml_gelu", g.tensor(ref.F32, allx)), out_shape=allx.shape)
    assert np.array_equal(oracle.gelu(allx), want_all)
    x64 = x.astype(np.float64)
    exact = 0.5 * x64 * (1 + np.tanh(np.sqrt(2 / np.pi) * x64 * (1 + 0.044715 * x64 ** 2)))
    assert oracle.nmse(got, exact) < 1e-6


@pytest.mark.parametrize("op", [0, 1])
def test_binary_broadcast(oracle, ref, op):
    a = rnd((3, 5, 16))
    for bshape in [(3, 5, 16), (16,), (1, 5, 1), (3, 1, 16)]:
        b = rnd(bshape)
        got = oracle.binary(op, a, b)
        want = a + b if op == 0 else a * b
        assert np.array_equal(got, want.astype(np.float32))
    with ref.Graph() as g:     # conv bias: [1, d] against [3000, d], repeated along ne0
        x, bias = rnd((6, 40)), rnd((6, 1))
        got_ref = g.run(g.op("ggml_add" if op == 0 else "ggml_mul", g.tensor(ref.F32, x), g.tensor(ref.F32, bias)), out_shape=x.shape)
    assert np.array_equal(oracle.binary(op, x, bias), got_ref)


def test_scale_softmax_im2col_get_rows(oracle, ref):
    x = rnd((4, 6, 50), 3.0)
    assert np.array_equal(oracle.scale(x, 0.35355339), (x * np.float32(0.35355339)).astype(np.float32))
    # softmax with and without mask
    mask = np.zeros((64, 50), dtype=np.float32)
    mask[:, 40:] = -np.inf
    for m in (None, mask):
        got = oracle.soft_max(x, None if m is None else m[:6], 0.125)
        with ref.Graph() as g:
            tm = g.tensor(ref.F32, m) if m is not None else None
            want = g.run(g.op("ggml_soft_max_ext", g.tensor(ref.F32, x), tm, 0.125, 0.0), out_shape=x.shape)
        assert oracle.nmse(got, want) < 1e-12
        z = x.astype(np.float64) * 0.125 + (0 if m is None else m[:6].astype(np.float64))
        e = np.exp(z - z.max(-1, keepdims=True))
        assert oracle.nmse(got, e / e.sum(-1, keepdims=True)) < 1e-12
        assert np.allclose(got.sum(-1), 1, atol=1e-6)
    # im2col, both strides of the conv stem
    src = rnd((5, 31))
    for s0 in (1, 2):
        got = oracle.im2col_1d(src, 3, s0, 1, 1)
        with ref.Graph() as g:
            w = g.tensor(ref.F16, np.zeros((2, 5, 3), dtype=np.uint16))
            want = g.run(g.op("ggml_im2col", w, g.tensor(ref.F32, src), s0, 0, 1, 0, 1, 0, False, ref.F16), out_type=ref.F16, out_shape=got.shape)
        assert np.array_equal(got, want)
        ow = got.shape[0]
        for o in range(ow):                       # closed form
            for ic in range(5):
                for kw in range(3):
                    iw = o * s0 + kw - 1
                    want_v = 0 if iw < 0 or iw >= 31 else oracle.f32_to_f16_bits(src[ic, iw : iw + 1])[0]
                    assert got[o, ic * 3 + kw] == want_v
    # get_rows = dequantization of the selected rows
    w = rnd((20, 64), 0.02)
    ids = np.array([3, 0, 19, 3], dtype=np.int32)
    for t in (oracle.Q5_0, oracle.Q8_0):
        blocks = oracle.quantize(t, w)
        got = oracle.get_rows(t, blocks, ids, 64)
        assert np.array_equal(got, oracle.dequantize(t, blocks, 64)[ids])
        with ref.Graph() as g:
            want = g.run(g.op("ggml_get_rows", g.tensor(t, blocks, ne=[64, 20]), g.tensor(ref.I32, ids)), out_shape=(4, 64))
        assert np.array_equal(got, want)


# ------------------------------------------------------------------------------------------------------------------
# log-mel front end
# ------------------------------------------------------------------------------------------------------------------

def mel_closed_form(samples, filters):
    """the same quantity from numpy's float64 rfft, with none of the reference's structure"""
    s = np.asarray(samples, dtype=np.float64)
    padded = np.concatenate([s[200:0:-1], s, np.zeros(480000 + 200)])
    n_len = (s.size + 480000) // 160
    idx = 160 * np.arange(n_len)[:, None] + np.arange(400)[None, :]
    window = 0.5 * (1.0 - np.cos(2.0 * np.pi * np.arange(400) / 400.0))
    power = np.abs(np.fft.rfft(padded[idx] * window, axis=1)) ** 2            # [n_len, 201]
    mel = np.log10(np.maximum(np.asarray(filters, dtype=np.float64) @ power.T, 1e-10))
    mel = np.maximum(mel, mel.max() - 8.0)
    return (mel + 4.0) / 4.0


def test_log_mel_against_float64_rfft(oracle):
    n = 16000 + 321
    t = np.arange(n) / 16000.0
    s = (0.25 * np.sin(2 * np.pi * 1000.0 * t) + 0.05 * RNG.normal(size=n)).astype(np.float32)
    f = oracle.mel_filter_bank(80)
    got, want = oracle.log_mel_spectrogram(s, f), mel_closed_form(s, f)
    assert got.shape == want.shape == (80, (n + 480000) // 160)
    # f32 transform against f64: the noise floor keeps every band well above the f32 rounding of the strongest one
    assert np.max(np.abs(got - want)) <= 2e-4
    # frames beyond the signal hold the clamp value; the band of the tone holds the maximum
    assert np.all(got[:, 110:] == got[0, 200])
    band = int(np.argmax(f[:, 25]))                       # bin 25 = 1000 Hz
    assert int(np.argmax(got[:, 50])) == band
    assert np.isclose(got.max(), (np.log10((f.astype(np.float64) @ (np.abs(np.fft.rfft(np.concatenate([s[200:0:-1], s])[160 * 50: 160 * 50 + 400].astype(np.float64)
                      * (0.5 - 0.5 * np.cos(2 * np.pi * np.arange(400) / 400)))) ** 2)).max()) + 4.0) / 4.0, atol=0.05)


def test_log_mel_against_the_reference(oracle, ref):
    if not ref.log_mel_available():
        pytest.skip("oracle/_ref/libref_mel.so is not built")
    for n, n_mel in ((4000 + 7, 80), (16000 * 2, 128), (201, 80)):
        t = np.arange(n) / 16000.0
        s = (0.5 * np.sin(2 * np.pi * (200.0 + 3000.0 * t) * t) + 0.02 * RNG.normal(size=n)).astype(np.float32)
        f = oracle.mel_filter_bank(n_mel)
        got, want = oracle.log_mel_spectrogram(s, f), ref.log_mel_spectrogram(s, f, n_threads=3)
        assert got.shape == want.shape
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))

"""numpy front end of oracle_ops.c — the CPU restatement of ggml's CPU-backend arithmetic.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py as the
checker; never by the product path.  All arrays are dense, row-major, with ggml's convention that the first
ggml dimension (ne0) is the fastest-varying one: a ggml tensor [ne0, ne1] is a numpy array of shape (ne1, ne0).
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "liboracle_ops.so"

F32, F16, Q5_0, Q8_0, I32 = 0, 1, 6, 8, 26
BLOCK_BYTES = {Q5_0: 22, Q8_0: 34}


def build() -> Path:
    """gcc the restatement into oracle/liboracle_ops.so (FMA contraction off: products and sums round separately)."""
    subprocess.run(["gcc", "-O2", "-std=gnu11", "-fPIC", "-shared", "-ffp-contract=off", "-o", str(LIB_PATH),
                    str(HERE / "oracle_ops.c"), "-lm"], check=True)
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        _lib = C.CDLL(str(LIB_PATH))
        _lib.oracle_f16_to_f32.restype = C.c_float
        _lib.oracle_f16_to_f32.argtypes = [C.c_uint16]
        _lib.oracle_f32_to_f16.restype = C.c_uint16
        _lib.oracle_f32_to_f16.argtypes = [C.c_float]
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def row_bytes(wtype: int, k: int) -> int:
    if wtype in BLOCK_BYTES:
        return k // 32 * BLOCK_BYTES[wtype]
    return k * (2 if wtype == F16 else 4)


# --- conversions / quantizers ---------------------------------------------------------------------------------

def f32_to_f16_bits(x) -> np.ndarray:
    x = _f32(x)
    y = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_f32_to_f16_row(_p(x), _p(y), C.c_int64(x.size))
    return y


def f16_bits_to_f32(h) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    y = np.empty(h.shape, dtype=np.float32)
    lib().oracle_f16_to_f32_row(_p(h), _p(y), C.c_int64(h.size))
    return y


def quantize(wtype: int, x, act: bool = False) -> np.ndarray:
    """f32 rows -> block bytes.  act=True is the activation quantizer of MUL_MAT (Q8_0 only, rounds half to even)."""
    x = _f32(x)
    k = x.shape[-1]
    rows = x.size // k
    out = np.empty((rows, row_bytes(wtype, k)), dtype=np.uint8)
    fn = {(Q5_0, False): "oracle_quantize_row_q5_0_ref", (Q8_0, False): "oracle_quantize_row_q8_0_ref",
          (Q8_0, True): "oracle_quantize_row_q8_0_act"}[(wtype, act)]
    getattr(lib(), fn)(_p(x), _p(out), C.c_int64(x.size))
    return out.reshape(x.shape[:-1] + (out.shape[1],))


def dequantize(wtype: int, blocks, k: int) -> np.ndarray:
    b = np.ascontiguousarray(blocks, dtype=np.uint8)
    rows = b.size // row_bytes(wtype, k)
    y = np.empty((rows, k), dtype=np.float32)
    fn = {Q5_0: "oracle_dequantize_row_q5_0", Q8_0: "oracle_dequantize_row_q8_0"}[wtype]
    getattr(lib(), fn)(_p(b), _p(y), C.c_int64(rows * k))
    return y.reshape(b.shape[:-1] + (k,))


# --- ops -----------------------------------------------------------------------------------------------------------

def mul_mat(wtype: int, w, x) -> np.ndarray:
    """w: [M, K] (f32 / f16-bit uint16 / block bytes [M, row_bytes]), x: f32 [N, K] -> f32 [N, M]"""
    x = _f32(x)
    n, k = x.shape
    w = np.ascontiguousarray(w)
    m = w.shape[0]
    dst = np.empty((n, m), dtype=np.float32)
    lib().oracle_mul_mat(C.c_int(wtype), _p(w), _p(x), _p(dst), C.c_int64(m), C.c_int64(n), C.c_int64(k))
    return dst


def mul_mat_f16_f16(a_bits, b_bits) -> np.ndarray:
    a = np.ascontiguousarray(a_bits, dtype=np.uint16)
    b = np.ascontiguousarray(b_bits, dtype=np.uint16)
    m, k = a.shape
    n = b.shape[0]
    dst = np.empty((n, m), dtype=np.float32)
    lib().oracle_mul_mat_f16_f16(_p(a), _p(b), _p(dst), C.c_int64(m), C.c_int64(n), C.c_int64(k))
    return dst


def flash_attn_ext(q, k_bits, v_bits, mask_bits, scale: float) -> np.ndarray:
    """q f32 [H, N, D], k/v f16 bits [H, KV, D], mask f16 bits [N, KV] or None -> f32 [N, H, D]"""
    q = _f32(q)
    k = np.ascontiguousarray(k_bits, dtype=np.uint16)
    v = np.ascontiguousarray(v_bits, dtype=np.uint16)
    h, n, d = q.shape
    kv = k.shape[1]
    m = None if mask_bits is None else np.ascontiguousarray(mask_bits, dtype=np.uint16)
    dst = np.empty((n, h, d), dtype=np.float32)
    lib().oracle_flash_attn_ext(_p(q), _p(k), _p(v), _p(m) if m is not None else None, _p(dst),
       C.c_int64(n), C.c_int64(kv), C.c_int64(h), C.c_int64(d), C.c_float(scale))
    return dst


def norm(x, eps: float) -> np.ndarray:
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_norm(_p(x), _p(y), C.c_int64(x.shape[-1]), C.c_int64(x.size // x.shape[-1]), C.c_float(eps))
    return y


def gelu(x) -> np.ndarray:
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_gelu(_p(x), _p(y), C.c_int64(x.size))
    return y


def binary(op: int, a, b) -> np.ndarray:
    """a, b: numpy arrays of up to 4 dims (numpy order = ggml order reversed); b's dims divide a's"""
    a = _f32(a)
    b = _f32(b)
    ane = (C.c_int64 * 4)(*([1] * (4 - a.ndim) + list(a.shape))[::-1])
    bne = (C.c_int64 * 4)(*([1] * (4 - b.ndim) + list(b.shape))[::-1])
    dst = np.empty_like(a)
    lib().oracle_binary(C.c_int(op), _p(a), ane, _p(b), bne, _p(dst))
    return dst


def scale(x, s: float) -> np.ndarray:
    x = _f32(x)
    y = np.empty_like(x)
    lib().oracle_scale(_p(x), _p(y), C.c_int64(x.size), C.c_float(s))
    return y


def im2col_1d(src, kw: int, s0: int, p0: int, d0: int) -> np.ndarray:
    """src f32 [IC, IW] -> f16 bits [OW, IC*KW]"""
    src = _f32(src)
    ic, iw = src.shape
    ow = (iw + 2 * p0 - d0 * (kw - 1) - 1) // s0 + 1
    dst = np.empty((ow, ic * kw), dtype=np.uint16)
    lib().oracle_im2col_1d(_p(src), _p(dst), C.c_int64(iw), C.c_int64(ic), C.c_int64(ow), C.c_int(kw), C.c_int(s0), C.c_int(p0), C.c_int(d0))
    return dst


def soft_max(x, mask, scale_: float) -> np.ndarray:
    """x f32 [..., rows, ne0]; mask f32 [rows, ne0] shared by all leading slices, or None"""
    x = _f32(x)
    y = np.empty_like(x)
    ne0 = x.shape[-1]
    rows = x.shape[-2] if x.ndim > 1 else 1
    m = None if mask is None else _f32(mask)
    lib().oracle_soft_max(_p(x), _p(m) if m is not None else None, _p(y), C.c_int64(ne0), C.c_int64(x.size // ne0), C.c_int64(rows), C.c_float(scale_))
    return y


def get_rows(wtype: int, table, ids, ne0: int) -> np.ndarray:
    t = np.ascontiguousarray(table)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    dst = np.empty((ids.size, ne0), dtype=np.float32)
    lib().oracle_get_rows(C.c_int(wtype), _p(t), _p(ids), _p(dst), C.c_int64(ne0), C.c_int64(ids.size))
    return dst


def nmse(got, want) -> float:
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    den = float(np.sum(want * want))
    num = float(np.sum((got - want) ** 2))
    return num / den if den > 0 else (0.0 if num == 0 else float("inf"))


def log_mel_spectrogram(samples, filters) -> np.ndarray:
    """samples f32 [n] at 16 kHz, filters f32 [n_mel, 201] -> mel f32 [n_mel, (n + 480000) // 160]"""
    s = _f32(samples).ravel()
    f = _f32(filters)
    assert s.size > 200 and f.ndim == 2 and f.shape[1] == 201
    L = lib()
    L.oracle_log_mel_n_len.restype = C.c_int64
    L.oracle_log_mel_spectrogram.restype = C.c_int64
    n_len = L.oracle_log_mel_n_len(C.c_int64(s.size))
    mel = np.empty((f.shape[0], n_len), dtype=np.float32)
    got = L.oracle_log_mel_spectrogram(_p(s), C.c_int64(s.size), _p(f), C.c_int(f.shape[0]), _p(mel))
    assert got == n_len
    return mel


def mel_filter_bank(n_mel: int, n_fft: int = 400, sample_rate: int = 16000) -> np.ndarray:
    """A triangular filter bank on the mel scale with area normalization, [n_mel, n_fft // 2 + 1] f32: synthetic test
    input of the kind a model file carries (the checks do not depend on its exact values)."""
    def hz_to_mel(f):
        return 2595.0 * np.log10(1.0 + np.asarray(f, dtype=np.float64) / 700.0)
    def mel_to_hz(m):
        return 700.0 * (10.0 ** (np.asarray(m, dtype=np.float64) / 2595.0) - 1.0)
    freqs = np.linspace(0.0, sample_rate / 2, n_fft // 2 + 1)
    edges = mel_to_hz(np.linspace(hz_to_mel(0.0), hz_to_mel(sample_rate / 2), n_mel + 2))
    bank = np.zeros((n_mel, freqs.size))
    for j in range(n_mel):
        lo, mid, hi = edges[j], edges[j + 1], edges[j + 2]
        up, down = (freqs - lo) / (mid - lo), (hi - freqs) / (hi - mid)
        bank[j] = np.maximum(0.0, np.minimum(up, down)) * 2.0 / (hi - lo)
    return bank.astype(np.float32)

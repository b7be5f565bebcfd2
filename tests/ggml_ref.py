"""ctypes access to the reference's own compiled code (oracle/_ref, built from /root/reference by oracle/Makefile):
libggml-base.so for the quantizers and graph construction, libggml-cpu.so for the CPU backend.

Test infrastructure: lets a pytest build a one-op ggml graph, run it on ggml's CPU backend and read the result as a
numpy array, so that the restatement in oracle/oracle_ops.c can be pinned against the real thing.  numpy arrays use
the reversed dimension order of ggml (a ggml tensor [ne0, ne1, ne2] is a numpy array of shape (ne2, ne1, ne0)).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
REF_DIR = ROOT / "oracle" / "_ref"

F32, F16, Q5_0, Q8_0, I32 = 0, 1, 6, 8, 26
NP_OF = {F32: np.float32, F16: np.uint16, I32: np.int32}


def available() -> bool:
    return (REF_DIR / "libggml-cpu.so").exists() and (REF_DIR / "libggml-base.so").exists()


class _InitParams(C.Structure):
    _fields_ = [("mem_size", C.c_size_t), ("mem_buffer", C.c_void_p), ("no_alloc", C.c_bool)]


_libs = None


def libs():
    global _libs
    if _libs is None:
        base = C.CDLL(str(REF_DIR / "libggml-base.so"), mode=C.RTLD_GLOBAL)
        cpu = C.CDLL(str(REF_DIR / "libggml-cpu.so"), mode=C.RTLD_GLOBAL)
        P = C.c_void_p
        base.ggml_init.restype = P
        base.ggml_init.argtypes = [_InitParams]
        base.ggml_free.argtypes = [P]
        base.ggml_tensor_overhead.restype = C.c_size_t
        base.ggml_graph_overhead.restype = C.c_size_t
        base.ggml_nbytes.restype = C.c_size_t
        base.ggml_nbytes.argtypes = [P]
        base.ggml_new_tensor.restype = P
        base.ggml_new_tensor.argtypes = [P, C.c_int, C.c_int, C.POINTER(C.c_int64)]
        for name, args in {
            "ggml_mul_mat": [P, P, P], "ggml_add": [P, P, P], "ggml_mul": [P, P, P], "ggml_gelu": [P, P],
            "ggml_scale": [P, P, C.c_float], "ggml_norm": [P, P, C.c_float], "ggml_get_rows": [P, P, P],
            "ggml_soft_max_ext": [P, P, P, C.c_float, C.c_float],
            "ggml_flash_attn_ext": [P, P, P, P, P, C.c_float, C.c_float, C.c_float],
            "ggml_im2col": [P, P, P, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_bool, C.c_int],
            "ggml_cast": [P, P, C.c_int], "ggml_cont": [P, P], "ggml_transpose": [P, P],
            "ggml_permute": [P, P, C.c_int, C.c_int, C.c_int, C.c_int],
        }.items():
            fn = getattr(base, name)
            fn.restype = P
            fn.argtypes = args
        base.ggml_new_graph.restype = P
        base.ggml_new_graph.argtypes = [P]
        base.ggml_build_forward_expand.argtypes = [P, P]
        base.ggml_backend_alloc_ctx_tensors.restype = P
        base.ggml_backend_alloc_ctx_tensors.argtypes = [P, P]
        base.ggml_backend_tensor_set.argtypes = [P, P, C.c_size_t, C.c_size_t]
        base.ggml_backend_tensor_get.argtypes = [P, P, C.c_size_t, C.c_size_t]
        base.ggml_backend_graph_compute.restype = C.c_int
        base.ggml_backend_graph_compute.argtypes = [P, P]
        base.ggml_backend_buffer_free.argtypes = [P]
        base.ggml_backend_free.argtypes = [P]
        base.ggml_quantize_chunk.restype = C.c_size_t
        base.ggml_quantize_chunk.argtypes = [C.c_int, P, P, C.c_int64, C.c_int64, C.c_int64, P]
        base.dequantize_row_q5_0.argtypes = [P, P, C.c_int64]
        base.dequantize_row_q8_0.argtypes = [P, P, C.c_int64]
        base.ggml_fp32_to_fp16_row.argtypes = [P, P, C.c_int64]
        base.ggml_fp16_to_fp32_row.argtypes = [P, P, C.c_int64]
        cpu.ggml_backend_cpu_init.restype = P
        cpu.ggml_backend_cpu_set_n_threads.argtypes = [P, C.c_int]
        cpu.quantize_row_q8_0.argtypes = [P, P, C.c_int64]
        # the first ggml_init fills the f16 -> f32 lookup table that GGML_FP16_TO_FP32 reads in the non-F16C objects
        base.ggml_free(base.ggml_init(_InitParams(1024, None, False)))
        _libs = (base, cpu)
    return _libs


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def row_bytes(t: int, k: int) -> int:
    return {F32: 4 * k, F16: 2 * k, I32: 4 * k, Q5_0: k // 32 * 22, Q8_0: k // 32 * 34}[t]


# --- quantizers of the reference ---------------------------------------------------------------------------------

def quantize_chunk(t: int, x: np.ndarray) -> np.ndarray:
    """ggml_quantize_chunk (ggml/src/ggml.c) on f32 rows -> block bytes"""
    base, _ = libs()
    x = np.ascontiguousarray(x, dtype=np.float32)
    k = x.shape[-1]
    rows = x.size // k
    out = np.empty((rows, row_bytes(t, k)), dtype=np.uint8)
    base.ggml_quantize_chunk(t, _ptr(x), _ptr(out), 0, rows, k, None)
    return out


def dequantize_row(t: int, blocks: np.ndarray, k: int) -> np.ndarray:
    base, _ = libs()
    b = np.ascontiguousarray(blocks, dtype=np.uint8)
    n = b.size // row_bytes(t, k) * k
    y = np.empty(n, dtype=np.float32)
    (base.dequantize_row_q5_0 if t == Q5_0 else base.dequantize_row_q8_0)(_ptr(b), _ptr(y), n)
    return y.reshape(-1, k)


def quantize_row_q8_0_cpu(x: np.ndarray) -> np.ndarray:
    """the CPU backend's activation quantizer (ggml-cpu-quants.c:738)"""
    _, cpu = libs()
    x = np.ascontiguousarray(x, dtype=np.float32)
    k = x.shape[-1]
    out = np.empty((x.size // k, row_bytes(Q8_0, k)), dtype=np.uint8)
    for r in range(out.shape[0]):
        cpu.quantize_row_q8_0(_ptr(x.reshape(-1, k)[r]), _ptr(out[r]), k)
    return out


def fp32_to_fp16(x: np.ndarray) -> np.ndarray:
    base, _ = libs()
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, dtype=np.uint16)
    base.ggml_fp32_to_fp16_row(_ptr(x), _ptr(y), x.size)
    return y


def fp16_to_fp32(h: np.ndarray) -> np.ndarray:
    base, _ = libs()
    h = np.ascontiguousarray(h, dtype=np.uint16)
    y = np.empty(h.shape, dtype=np.float32)
    base.ggml_fp16_to_fp32_row(_ptr(h), _ptr(y), h.size)
    return y


# --- one-op graphs on the CPU backend ---------------------------------------------------------------------------

class Graph:
    """build tensors with .tensor(), combine them with the ggml_* constructors through .op(), then .run(result)"""

    def __init__(self, threads: int = 4):
        self.base, self.cpu = libs()
        params = _InitParams(self.base.ggml_tensor_overhead() * 64 + self.base.ggml_graph_overhead(), None, True)
        self.ctx = self.base.ggml_init(params)
        self.backend = self.cpu.ggml_backend_cpu_init()
        self.cpu.ggml_backend_cpu_set_n_threads(self.backend, threads)
        self.pending = []          # (tensor, numpy data)
        self.buf = None

    def tensor(self, t: int, data: np.ndarray, ne=None):
        """new leaf holding `data`; for block types pass ne (ggml order) explicitly"""
        data = np.ascontiguousarray(data)
        if ne is None:
            ne = list(data.shape)[::-1]
        dims = (C.c_int64 * len(ne))(*ne)
        tp = self.base.ggml_new_tensor(self.ctx, t, len(ne), dims)
        self.pending.append((tp, data))
        return tp

    def op(self, name: str, *args):
        return getattr(self.base, name)(self.ctx, *args)

    def run(self, result, out_type: int = F32, out_shape=None) -> np.ndarray:
        gf = self.base.ggml_new_graph(self.ctx)
        self.base.ggml_build_forward_expand(gf, result)
        self.buf = self.base.ggml_backend_alloc_ctx_tensors(self.ctx, self.backend)
        assert self.buf, "allocation failed"
        for tp, data in self.pending:
            nbytes = self.base.ggml_nbytes(tp)
            assert nbytes == data.nbytes, (nbytes, data.nbytes)
            self.base.ggml_backend_tensor_set(tp, _ptr(data), 0, nbytes)
        status = self.base.ggml_backend_graph_compute(self.backend, gf)
        assert status == 0, status
        nbytes = self.base.ggml_nbytes(result)
        out = np.empty(nbytes // np.dtype(NP_OF[out_type]).itemsize, dtype=NP_OF[out_type])
        self.base.ggml_backend_tensor_get(result, _ptr(out), 0, nbytes)
        return out.reshape(out_shape) if out_shape is not None else out

    def close(self):
        if self.buf:
            self.base.ggml_backend_buffer_free(self.buf)
        self.base.ggml_backend_free(self.backend)
        self.base.ggml_free(self.ctx)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


# --- the reference's log-mel front end (oracle/ref_mel_shim.cpp -> oracle/_ref/libref_mel.so) ----------------------

def log_mel_available() -> bool:
    return (REF_DIR / "libref_mel.so").exists()


_mel_lib = None


def log_mel_spectrogram(samples: np.ndarray, filters: np.ndarray, n_threads: int = 4) -> np.ndarray:
    """log_mel_spectrogram (src/whisper.cpp:3181-3270) on f32 samples and a [n_mel, 201] filter bank -> [n_mel, n_len]"""
    global _mel_lib
    if _mel_lib is None:
        _mel_lib = C.CDLL(str(REF_DIR / "libref_mel.so"))
    s = np.ascontiguousarray(samples, dtype=np.float32).ravel()
    f = np.ascontiguousarray(filters, dtype=np.float32)
    n_len = C.c_int()
    assert _mel_lib.ref_log_mel_spectrogram(_ptr(s), C.c_int(s.size), _ptr(f), C.c_int(f.shape[0]), C.c_int(n_threads), None, C.c_int(0), C.byref(n_len), None) == 0
    out = np.empty((f.shape[0], n_len.value), dtype=np.float32)
    assert _mel_lib.ref_log_mel_spectrogram(_ptr(s), C.c_int(s.size), _ptr(f), C.c_int(f.shape[0]), C.c_int(n_threads), _ptr(out), C.c_int(out.size), None, None) == 0
    return out

"""ggml-mi355x: a from-scratch MI355X (gfx950) compute backend for ggml / whisper.cpp.

The product is native: ``lib/libmi355x_kernels.so`` (hand-written HIP kernels behind the C ABI of
``include/mi355x_kernels.h``) and ``lib/libggml-mi355x.so`` (the ggml backend plugin, ``include/ggml-mi355x.h``).
This Python package is a thin ctypes view of the kernel ABI — used by the tests, the smoke check and the bench
to drive the kernels with device memory owned by PyTorch — plus the build recipes (``build.py``).

There is no CPU fallback: everything here raises if the HIP library has not been built or no GPU is present.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
LIB_DIR = PKG_DIR / "lib"
KERNELS_LIB = LIB_DIR / "libmi355x_kernels.so"
PLUGIN_LIB = LIB_DIR / "libggml-mi355x.so"
HARNESS_BIN = LIB_DIR / "mi355x-harness"

# enum mi355x_type (numeric values of the reference's enum ggml_type)
F32, F16, Q5_0, Q8_0, I32 = 0, 1, 6, 8, 26
BLOCK_BYTES = {Q5_0: 22, Q8_0: 34}

# enum mi355x_epilogue_flags
EPI_BIAS, EPI_GELU, EPI_SCALE, EPI_RESIDUAL, EPI_BIAS_COL, EPI_OUT_F16 = 1, 2, 4, 8, 16, 32
MM_EXACT_ACT, MM_WS_READY, MM_ACT_Q8_0, MM_PREPARE_ONLY, EPI_EMIT_F16, EPI_IMAGE_ONLY, EPI_EMIT_Q8_0 = 64, 128, 256, 512, 1024, 2048, 4096
MUL_MAT_NOALLOC_MAX = 32 << 20
# enum mi355x_fa_mode
FA_F16_SEQ, FA_F32, FA_F16_PK, FA_EMIT_F16, FA_EMIT_Q8_0 = 0, 1, 2, 0x100, 0x200


class Tensor(C.Structure):
    """struct mi355x_tensor"""
    _fields_ = [("data", C.c_void_p), ("type", C.c_int32), ("_pad", C.c_int32), ("ne", C.c_int64 * 4), ("nb", C.c_size_t * 4)]


class Epilogue(C.Structure):
    """struct mi355x_epilogue"""
    _fields_ = [("flags", C.c_int32), ("scale", C.c_float), ("bias", C.c_void_p), ("residual", C.c_void_p), ("image", C.c_void_p)]


class MulMatItem(C.Structure):
    """struct mi355x_mul_mat_item"""
    _fields_ = [("src0", C.POINTER(Tensor)), ("dst", C.POINTER(Tensor)), ("epi", C.POINTER(Epilogue))]


class MissingExtension(RuntimeError):
    pass


_lib = None


def kernels() -> C.CDLL:
    """The kernel library.  Raises MissingExtension when it has not been built: there is no other compute path."""
    global _lib
    if _lib is None:
        if not KERNELS_LIB.exists():
            raise MissingExtension(f"{KERNELS_LIB} is missing: build it with `python whisper.cpp_amd/build.py` (or __graft_entry__.build())")
        lib = C.CDLL(str(KERNELS_LIB))
        P, T = C.c_void_p, C.POINTER(Tensor)
        sig = {
            "mi355x_abi_version": (C.c_int, []),
            "mi355x_device_is_gfx950": (C.c_int, [C.c_int]),
            "mi355x_status_string": (C.c_char_p, [C.c_int]),
            "mi355x_dequantize_row": (C.c_int, [C.c_int, P, P, C.c_int64, P]),
            "mi355x_dequantize_row_f16": (C.c_int, [C.c_int, P, P, C.c_int64, P]),
            "mi355x_quantize_row_q8_0": (C.c_int, [P, P, C.c_int64, P]),
            "mi355x_mul_mat_kernel_name": (C.c_char_p, [T, T]),
            "mi355x_mul_mat_workspace_size": (C.c_size_t, [T, T]),
            "mi355x_mul_mat": (C.c_int, [T, T, T, C.POINTER(Epilogue), P, C.c_size_t, P]),
            "mi355x_mul_mat_noalloc": (C.c_int, [T, T, T, C.POINTER(Epilogue), P]),
            "mi355x_mul_mat_group": (C.c_int, [C.POINTER(MulMatItem), C.c_int, T, C.c_int, P, C.c_size_t, P]),
            "mi355x_q8_0_tiles_size": (C.c_size_t, [C.c_int64, C.c_int64]),
            "mi355x_q8_0_tiles_pack": (C.c_int, [T, P, P]),
            "mi355x_mul_mat_q8_0_tiles": (C.c_int, [P, C.c_int64, C.c_int64, T, T, C.c_int, P, C.c_size_t, P]),
            "mi355x_norm_mul_mat_q8_0_tiles": (C.c_int, [P, C.c_int64, C.c_int64, T, T, C.c_float, P, P, T, C.c_int, P, C.c_size_t, P]),
            "mi355x_norm_mul_mat_group": (C.c_int, [T, T, C.c_float, P, P, C.POINTER(MulMatItem), C.c_int, P, C.c_size_t, P]),
            "mi355x_embed_norm_mul_mat_group": (C.c_int, [T, T, T, T, T, T, C.c_float, P, P, C.POINTER(MulMatItem), C.c_int, P, C.c_size_t, P]),
            "mi355x_flash_attn_ext_kernel_name": (C.c_char_p, [T, T, C.c_int]),
            "mi355x_flash_attn_ext_workspace_size": (C.c_size_t, [T, T]),
            "mi355x_flash_attn_ext": (C.c_int, [T, T, T, T, T, C.c_float, C.c_int, P, C.c_size_t, P]),
            "mi355x_flash_attn_ext_cast_mask": (C.c_int, [T, T, T, T, T, T, C.c_float, C.c_int, P, C.c_size_t, P]),
            "mi355x_binary": (C.c_int, [C.c_int, T, T, T, P]),
            "mi355x_scale": (C.c_int, [T, T, C.c_float, P]),
            "mi355x_gelu": (C.c_int, [T, T, P]),
            "mi355x_norm": (C.c_int, [T, T, C.c_float, P, P, P]),
            "mi355x_norm_emit_f16": (C.c_int, [T, T, C.c_float, P, P, P, P]),
            "mi355x_norm_emit_q8_0": (C.c_int, [T, T, C.c_float, P, P, P, P]),
            "mi355x_soft_max": (C.c_int, [T, T, T, C.c_float, P]),
            "mi355x_cpy": (C.c_int, [T, T, P]),
            "mi355x_get_rows": (C.c_int, [T, T, T, P]),
            "mi355x_get_rows_add": (C.c_int, [T, T, T, T, T, P]),
            "mi355x_im2col_1d": (C.c_int, [T, T, C.c_int, C.c_int, C.c_int, C.c_int, P]),
            "mi355x_concat": (C.c_int, [T, T, T, C.c_int, P]),
            "mi355x_fill_bytes": (C.c_int, [P, C.c_uint8, C.c_size_t, P]),
            "mi355x_log_mel_n_len": (C.c_int64, [C.c_int64]),
            "mi355x_log_mel_workspace_size": (C.c_size_t, [C.c_int]),
            "mi355x_log_mel_spectrogram": (C.c_int, [P, C.c_int64, P, C.c_int, P, P, C.c_size_t, P]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def row_bytes(ttype: int, ne0: int) -> int:
    if ttype in BLOCK_BYTES:
        return ne0 // 32 * BLOCK_BYTES[ttype]
    return ne0 * (2 if ttype == F16 else 4)


def tensor(t, ttype: int, ne=None, nb=None) -> Tensor:
    """Describe a torch CUDA tensor (or anything with data_ptr()) as a mi355x_tensor.

    ne / nb use ggml's order (ne[0] is the contiguous dimension).  Without ne/nb the torch tensor's own shape and
    strides are used, reversed; block-quantized data is passed as a uint8 tensor together with explicit ne.
    """
    out = Tensor()
    out.data = t.data_ptr()
    out.type = ttype
    if ne is None:
        ne = list(t.shape)[::-1]
        esz = t.element_size()
        nb = [s * esz for s in t.stride()][::-1]
    ne = list(ne) + [1] * (4 - len(ne))
    if nb is None:
        nb = [BLOCK_BYTES.get(ttype, 2 if ttype == F16 else 4), row_bytes(ttype, ne[0])]
        nb.append(nb[1] * ne[1])
        nb.append(nb[2] * ne[2])
    nb = list(nb)
    while len(nb) < 4:
        nb.append(nb[-1] * ne[len(nb) - 1])
    for i in range(4):
        out.ne[i] = ne[i]
        out.nb[i] = nb[i]
    return out


def check(status: int, what: str = "kernel") -> None:
    if status != 0:
        raise RuntimeError(f"{what}: {kernels().mi355x_status_string(status).decode()} ({status})")

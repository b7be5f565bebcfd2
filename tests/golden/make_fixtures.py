"""Writes tests/golden/*.npz: small input / expected-output vectors for every op of the path, computed by the
reference's own compiled code (oracle/_ref: libggml-base quantizers, one-op graphs on the ggml CPU backend).

Run in a container that has the reference built (python oracle/... make, see oracle/Makefile):
    python tests/golden/make_fixtures.py                    # cpu_backend_vectors.npz and log_mel_vectors.npz
    python tests/golden/make_fixtures.py --log-mel-only     # only log_mel_vectors.npz (the reference's log-mel front end,
                                                            # reached through oracle/ref_mel_shim.cpp)
The fixtures are data only; tests/test_golden.py checks the oracle restatement against them on the CPU, and
tests/test_kernels_gpu.py checks the HIP kernels against them on the GPU box, where the reference does not exist.
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent))
import ggml_ref as ref  # noqa: E402

rng = np.random.default_rng(424242)


def rnd(shape, scale=1.0, offset=0.0):
    return (rng.normal(size=shape) * scale + offset).astype(np.float32)


def main() -> None:
    assert ref.available(), "build oracle/_ref first (make -C oracle)"
    out = {}

    # block formats: model-file quantizers and dequantization (bit-exact contract)
    w = rnd((6, 128), 0.02)
    w[0, :32] = 0.0                       # an all-zero block
    w[1, 5] = 0.5                         # an outlier that sets the scale
    for name, t in (("q5_0", ref.Q5_0), ("q8_0", ref.Q8_0)):
        blocks = ref.quantize_chunk(t, w)
        out[f"quant_{name}_input"] = w
        out[f"quant_{name}_blocks"] = blocks
        out[f"dequant_{name}"] = ref.dequantize_row(t, blocks, 128)

    # the CPU backend's activation quantizer (AVX2 rounding)
    x = rnd((4, 96), 1.0)
    x[0, :8] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, 127.0]      # exact halves after scaling by 127/127
    out["act_q8_0_input"] = x
    out["act_q8_0_blocks"] = ref.quantize_row_q8_0_cpu(x)

    # MUL_MAT: quantized weights x f32 activations, GEMV (n = 1, 5) and GEMM (n = 40) widths
    for name, t in (("q5_0", ref.Q5_0), ("q8_0", ref.Q8_0)):
        k, m = 128, 48
        wf = rnd((m, k), 0.02)
        blocks = ref.quantize_chunk(t, wf)
        out[f"mul_mat_{name}_w"] = blocks
        for n in (1, 5, 40):
            xa = rnd((n, k), 1.0)
            with ref.Graph() as g:
                tw = g.tensor(t, blocks, ne=[k, m])
                tx = g.tensor(ref.F32, xa)
                y = g.run(g.op("ggml_mul_mat", tw, tx), out_shape=(n, m))
            out[f"mul_mat_{name}_x_n{n}"] = xa
            out[f"mul_mat_{name}_y_n{n}"] = y

    # FLASH_ATTN_EXT: encoder-like (no mask), decoder-like (causal mask with -inf, scale 1)
    for name, (h, n, kv, masked, scale) in {"enc": (2, 70, 100, False, 0.125), "dec": (3, 5, 37, True, 1.0)}.items():
        q = rnd((h, n, 64))
        kk = ref.fp32_to_fp16(rnd((h, kv, 64)))
        vv = ref.fp32_to_fp16(rnd((h, kv, 64), 1.0, 0.3))
        npad = (n + 63) // 64 * 64
        mask = None
        if masked:
            mf = np.zeros((npad, kv), dtype=np.float32)
            for i in range(n):
                mf[i, kv - n + i + 1:] = -np.inf
            mask = ref.fp32_to_fp16(mf)
        with ref.Graph() as g:
            tq = g.tensor(ref.F32, q)
            tk = g.tensor(ref.F16, kk)
            tv = g.tensor(ref.F16, vv)
            tm = g.tensor(ref.F16, mask) if mask is not None else None
            y = g.run(g.op("ggml_flash_attn_ext", tq, tk, tv, tm, np.float32(scale), np.float32(0.0), np.float32(0.0)), out_shape=(n, h, 64))
        out[f"fa_{name}_q"], out[f"fa_{name}_k"], out[f"fa_{name}_v"], out[f"fa_{name}_y"] = q, kk, vv, y
        out[f"fa_{name}_scale"] = np.float32(scale)
        if mask is not None:
            out[f"fa_{name}_mask"] = mask

    # NORM, GELU, SOFT_MAX
    xn = rnd((7, 384), 2.0, 0.5)
    with ref.Graph() as g:
        out["norm_y"] = g.run(g.op("ggml_norm", g.tensor(ref.F32, xn), np.float32(1e-5)), out_shape=xn.shape)
    out["norm_x"] = xn
    xg = np.concatenate([rnd((500,), 3.0), np.array([-11.0, -10.0, -9.99, 0.0, 9.99, 10.0, 11.0], dtype=np.float32)])
    with ref.Graph() as g:
        out["gelu_y"] = g.run(g.op("ggml_gelu", g.tensor(ref.F32, xg)), out_shape=xg.shape)
    out["gelu_x"] = xg
    xs = rnd((2, 5, 33), 2.0)
    with ref.Graph() as g:
        out["soft_max_y"] = g.run(g.op("ggml_soft_max_ext", g.tensor(ref.F32, xs), None, np.float32(0.7), np.float32(0.0)), out_shape=xs.shape)
    out["soft_max_x"] = xs
    out["soft_max_scale"] = np.float32(0.7)

    np.savez_compressed(HERE / "cpu_backend_vectors.npz", **out)
    total = sum(v.nbytes for v in out.values())
    print(f"wrote {len(out)} arrays, {total / 1024:.0f} KiB uncompressed")


def mel_signal(n: int, seed: int) -> np.ndarray:
    """tones, a chirp, a click and noise: energy in every part of the band, frames of very different level"""
    r = np.random.default_rng(seed)
    t = np.arange(n) / 16000.0
    s = 0.3 * np.sin(2 * np.pi * 440.0 * t) + 0.1 * np.sin(2 * np.pi * (500.0 + 9000.0 * t) * t) + 0.01 * r.normal(size=n)
    s[n // 3] += 0.9
    s[: n // 8] *= 1e-3
    return s.astype(np.float32)


def write_log_mel() -> None:
    """tests/golden/log_mel_vectors.npz: the reference's log-mel front end on two short signals.  Frames beyond the
    signal all hold one value, so only the leading frames and that value are kept."""
    assert ref.log_mel_available(), "build oracle/_ref first (make -C oracle)"
    sys.path.insert(0, str(HERE.parent.parent / "oracle"))
    import oracle
    out = {}
    for name, n, n_mel, seed in (("a", 16000 + 123, 80, 7), ("b", 8000 + 1, 128, 8)):
        s = mel_signal(n, seed)
        f = oracle.mel_filter_bank(n_mel)
        mel = ref.log_mel_spectrogram(s, f)
        keep = (n + 200) // 160 + 9
        assert np.all(mel[:, keep:] == mel[:, keep: keep + 1])
        out[f"mel_{name}_samples"] = s
        out[f"mel_{name}_filters"] = f
        out[f"mel_{name}_head"] = mel[:, :keep].copy()
        out[f"mel_{name}_tail_value"] = mel[:, keep].copy()
        out[f"mel_{name}_n_len"] = np.int64(mel.shape[1])
    np.savez_compressed(HERE / "log_mel_vectors.npz", **out)
    print(f"wrote log_mel_vectors.npz: {sum(v.nbytes for v in out.values()) / 1024:.0f} KiB uncompressed")


if __name__ == "__main__":
    if "--log-mel-only" not in sys.argv:
        main()
    write_log_mel()

"""The committed vectors of tests/golden/cpu_backend_vectors.npz — inputs and the outputs the reference's own compiled
code (ggml-base quantizers, ggml CPU backend) gave for them, written by tests/golden/make_fixtures.py — against the
oracle restatement.  Runs without the reference and without a GPU; the GPU counterpart is in test_kernels_gpu.py."""
from __future__ import annotations

from pathlib import Path

import numpy as np
import pytest

GOLDEN = Path(__file__).resolve().parent / "golden" / "cpu_backend_vectors.npz"


@pytest.fixture(scope="module")
def vec():
    return np.load(GOLDEN, allow_pickle=False)


@pytest.mark.parametrize("name", ["q5_0", "q8_0"])
def test_block_formats_bit_exact(oracle, vec, name):
    t = getattr(oracle, name.upper())
    assert np.array_equal(oracle.quantize(t, vec[f"quant_{name}_input"]), vec[f"quant_{name}_blocks"])
    got = oracle.dequantize(t, vec[f"quant_{name}_blocks"], 128)
    assert np.array_equal(got.view(np.uint32), vec[f"dequant_{name}"].view(np.uint32))


def test_activation_quantizer_bit_exact(oracle, vec):
    assert np.array_equal(oracle.quantize(oracle.Q8_0, vec["act_q8_0_input"], act=True), vec["act_q8_0_blocks"])


@pytest.mark.parametrize("name", ["q5_0", "q8_0"])
@pytest.mark.parametrize("n", [1, 5, 40])
def test_mul_mat(oracle, vec, name, n):
    t = getattr(oracle, name.upper())
    got = oracle.mul_mat(t, vec[f"mul_mat_{name}_w"], vec[f"mul_mat_{name}_x_n{n}"])
    assert oracle.nmse(got, vec[f"mul_mat_{name}_y_n{n}"]) <= 1e-12      # same integers and scales, other summation order


@pytest.mark.parametrize("name", ["enc", "dec"])
def test_flash_attn(oracle, vec, name):
    q = vec[f"fa_{name}_q"]
    mask = vec[f"fa_{name}_mask"][: q.shape[1]] if f"fa_{name}_mask" in vec else None
    got = oracle.flash_attn_ext(q, vec[f"fa_{name}_k"], vec[f"fa_{name}_v"], mask, float(vec[f"fa_{name}_scale"]))
    assert oracle.nmse(got, vec[f"fa_{name}_y"]) <= 1e-7                # same f16 chain; the dot products sum in another order


def test_norm_gelu_soft_max(oracle, vec):
    assert oracle.nmse(oracle.norm(vec["norm_x"], 1e-5), vec["norm_y"]) <= 1e-12
    assert np.array_equal(oracle.gelu(vec["gelu_x"]), vec["gelu_y"])
    assert oracle.nmse(oracle.soft_max(vec["soft_max_x"], None, float(vec["soft_max_scale"])), vec["soft_max_y"]) <= 1e-12


# ------------------------------------------------------------------------------------------------------------------
# log-mel front end: tests/golden/log_mel_vectors.npz, written by the reference's compiled log_mel_spectrogram
# ------------------------------------------------------------------------------------------------------------------

MEL_GOLDEN = Path(__file__).resolve().parent / "golden" / "log_mel_vectors.npz"


def mel_cases():
    v = np.load(MEL_GOLDEN, allow_pickle=False)
    for name in ("a", "b"):
        head, tail = v[f"mel_{name}_head"], v[f"mel_{name}_tail_value"]
        want = np.empty((head.shape[0], int(v[f"mel_{name}_n_len"])), dtype=np.float32)
        want[:, :head.shape[1]] = head
        want[:, head.shape[1]:] = tail[:, None]
        yield name, v[f"mel_{name}_samples"], v[f"mel_{name}_filters"], want


@pytest.mark.parametrize("case", list(mel_cases()), ids=lambda c: c[0])
def test_log_mel_spectrogram(oracle, case):
    _, samples, filters, want = case
    got = oracle.log_mel_spectrogram(samples, filters)
    assert got.shape == want.shape
    # the restatement keeps the reference's f32 operation order (it was bit-equal where the vectors were written);
    # libm's sinf / cosf / log10 are the only parts that may differ between machines
    assert np.max(np.abs(got - want)) <= 1e-6

"""mi355x_mul_mat_noalloc — MUL_MAT for callers that cannot allocate device memory — against mi355x_mul_mat with a
workspace of the caller's, through the C ABI.  The two share their kernels, so the bar is bit equality.  Each case makes
two calls in a row on the library's fixed scratch array, the second with a smaller input, so that what the first left in
the array must not show in the second result."""
from __future__ import annotations

import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(11)


def rnd(shape, scale=1.0):
    return (RNG.normal(size=shape) * scale).astype(np.float32)


@pytest.fixture(scope="module")
def dev(pkg):
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the gpu-marked tests must run on the MI355X box")
    assert pkg.kernels().mi355x_device_is_gfx950(0) == 1
    return torch.device("cuda:0")


def operands(pkg, oracle, dev, wtype, k, m, n, flags):
    t = getattr(pkg, wtype)
    if t in pkg.BLOCK_BYTES:
        w = torch.from_numpy(oracle.quantize(t, rnd((m, k), 0.02))).to(dev)
    else:
        w = torch.from_numpy(rnd((m, k), 0.02)).to(dev)
    x = torch.from_numpy(rnd((n, k))).to(dev)
    keep = [w, x]
    epi = pkg.Epilogue()
    epi.flags, epi.scale = flags, 1.0
    if flags & pkg.EPI_BIAS:
        keep.append(torch.from_numpy(rnd((m,))).to(dev)); epi.bias = keep[-1].data_ptr()
    if flags & pkg.EPI_RESIDUAL:
        keep.append(torch.from_numpy(rnd((n, m))).to(dev)); epi.residual = keep[-1].data_ptr()
    return pkg.tensor(w, t, ne=[k, m]), pkg.tensor(x, pkg.F32), epi, keep


def both(pkg, dev, tw, tx, epi, n, m):
    """the product through mi355x_mul_mat (own workspace) and through mi355x_mul_mat_noalloc; returns the two results"""
    lib = pkg.kernels()
    stream = C.c_void_p(0)
    pe = C.byref(epi) if epi.flags else None
    y_ws = torch.full((n, m), float("nan"), dtype=torch.float32, device=dev)
    y_na = torch.full((n, m), float("nan"), dtype=torch.float32, device=dev)
    ws_size = lib.mi355x_mul_mat_workspace_size(tw, tx)
    assert ws_size <= pkg.MUL_MAT_NOALLOC_MAX
    ws = torch.empty(max(ws_size, 256), dtype=torch.uint8, device=dev)
    pkg.check(lib.mi355x_mul_mat(tw, tx, pkg.tensor(y_ws, pkg.F32), pe, ws.data_ptr(), ws_size, stream), "mul_mat")
    pkg.check(lib.mi355x_mul_mat_noalloc(tw, tx, pkg.tensor(y_na, pkg.F32), pe, stream), "mul_mat_noalloc")
    torch.cuda.synchronize()
    return y_ws.cpu().numpy(), y_na.cpu().numpy()


# (weight type, K, M, N of the first call, N of the second, epilogue): the many-column path (f16 images of both operands in
# the scratch array), the few-column path (Q8_0 activations there), an F32 weight matrix, and one without scratch at all
CASES = [
    ("Q5_0", 1280, 640, 300, 70, 0),
    ("Q8_0", 512, 2048, 1500, 33, 1 | 8),          # bias + residual
    ("Q8_0", 1280, 1280, 5, 2, 0),
    ("Q5_0", 5120, 1280, 8, 1, 1),
    ("F32", 256, 96, 40, 9, 0),
    ("Q8_0", 1280, 2048, 129, 5, 2),               # GELU epilogue; second call takes the few-column path on the same array
]


@pytest.mark.parametrize("case", CASES)
def test_noalloc_equals_mul_mat_on_two_calls_in_a_row(pkg, oracle, dev, case):
    wtype, k, m, n1, n2, flags = case
    for n in (n1, n2):
        print(f"mul_mat_noalloc case {wtype} K={k} M={m} N={n} flags={flags}", flush=True)
        tw, tx, epi, keep = operands(pkg, oracle, dev, wtype, k, m, n, flags)
        want, got = both(pkg, dev, tw, tx, epi, n, m)
        assert not np.isnan(want).any()
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), (case, n)


def test_noalloc_rejects_what_does_not_fit_and_what_relies_on_old_contents(pkg, oracle, dev):
    lib = pkg.kernels()
    stream = C.c_void_p(0)
    # 1500 x 5120 activations and a 5120 x 5120 Q5_0 matrix want 15 MB + 52 MB of scratch: beyond the 32 MiB array
    k, m, n = 5120, 5120, 1500
    w = torch.zeros(m * (k // 32) * 22, dtype=torch.uint8, device=dev)
    x = torch.zeros((n, k), dtype=torch.float32, device=dev)
    y = torch.zeros((n, m), dtype=torch.float32, device=dev)
    tw, tx, ty = pkg.tensor(w, pkg.Q5_0, ne=[k, m]), pkg.tensor(x, pkg.F32), pkg.tensor(y, pkg.F32)
    assert lib.mi355x_mul_mat_workspace_size(tw, tx) > pkg.MUL_MAT_NOALLOC_MAX
    assert lib.mi355x_mul_mat_noalloc(tw, tx, ty, None, stream) == -3          # MI355X_ERR_WORKSPACE
    # the array is shared: no call may say that it already holds its activations, or stop after writing them
    tw, tx, epi, keep = operands(pkg, oracle, dev, "Q8_0", 512, 256, 40, 0)
    y = torch.zeros((40, 256), dtype=torch.float32, device=dev)
    for flag in (pkg.MM_WS_READY, pkg.MM_PREPARE_ONLY):
        epi.flags = flag
        assert lib.mi355x_mul_mat_noalloc(tw, tx, pkg.tensor(y, pkg.F32), C.byref(epi), stream) == -2     # MI355X_ERR_INVALID
    assert lib.mi355x_mul_mat_noalloc(None, tx, pkg.tensor(y, pkg.F32), None, stream) == -2
    torch.cuda.synchronize()

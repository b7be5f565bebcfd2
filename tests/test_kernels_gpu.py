"""GPU parity of the HIP kernels, called through the C ABI of include/mi355x_kernels.h with device memory owned by
torch, against the CPU restatement in oracle/ on the same seeded inputs.

Bars: bit-exact for dequantization, gathers, copies/conversions, IM2COL and the f32 elementwise ops; for the
floating-point kernels the tolerance is written next to each check (the north-star per-op bound is NMSE <= 5e-4 against
the CPU backend; the reference-faithful paths are held to <= 1e-6)."""
from __future__ import annotations

import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(7)


def rnd(shape, scale=1.0, offset=0.0):
    return (RNG.normal(size=shape) * scale + offset).astype(np.float32)


@pytest.fixture(scope="module")
def gpu(pkg):
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the gpu-marked tests must run on the MI355X box")
    lib = pkg.kernels()
    assert lib.mi355x_device_is_gfx950(0) == 1

    class G:
        dev = torch.device("cuda:0")
        stream = C.c_void_p(0)

        @staticmethod
        def up(a: np.ndarray):
            a = np.ascontiguousarray(a)
            if a.dtype == np.uint16:
                a = a.view(np.int16)
            return torch.from_numpy(a).to(G.dev)

        @staticmethod
        def down(t, dtype=None):
            torch.cuda.synchronize()
            a = t.cpu().numpy()
            return a.view(dtype) if dtype is not None else a

    return G


def run_mul_mat(pkg, gpu, wtype, wdata, x, k, m, flags=0, bias=None, resid=None, scale=1.0, out_f16=False, workspace=True):
    lib = pkg.kernels()
    d_w, d_x = gpu.up(wdata), gpu.up(x)
    n = x.shape[0]
    d_y = torch.empty((n, m), dtype=torch.float16 if out_f16 else torch.float32, device=gpu.dev)
    tw = pkg.tensor(d_w, wtype, ne=[k, m])
    tx = pkg.tensor(d_x, pkg.F32)
    ty = pkg.tensor(d_y, pkg.F16 if out_f16 else pkg.F32)
    ws_size = lib.mi355x_mul_mat_workspace_size(tw, tx) if workspace else 0
    ws = torch.empty(max(ws_size, 16), dtype=torch.uint8, device=gpu.dev)
    epi = pkg.Epilogue()
    epi.flags, epi.scale = flags | (pkg.EPI_OUT_F16 if out_f16 else 0), scale
    keep = []
    if bias is not None:
        keep.append(gpu.up(bias)); epi.bias = keep[-1].data_ptr()
    if resid is not None:
        keep.append(gpu.up(resid)); epi.residual = keep[-1].data_ptr()
    pkg.check(lib.mi355x_mul_mat(tw, tx, ty, C.byref(epi) if epi.flags else None, ws.data_ptr(), ws_size, gpu.stream), "mul_mat")
    name = lib.mi355x_mul_mat_kernel_name(tw, tx).decode()
    return gpu.down(d_y).astype(np.float32), name


# ------------------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("wtype", ["Q5_0", "Q8_0"])
def test_dequantize_row_bit_exact(pkg, oracle, gpu, wtype):
    t = getattr(pkg, wtype)
    k = 32 * 4099                                        # odd number of blocks
    blocks = RNG.integers(0, 256, size=(k // 32, pkg.BLOCK_BYTES[t]), dtype=np.uint8)      # arbitrary bytes: every scale pattern incl. inf / nan / subnormal
    d_b = gpu.up(blocks)
    d_y = torch.empty(k, dtype=torch.float32, device=gpu.dev)
    pkg.check(pkg.kernels().mi355x_dequantize_row(t, d_b.data_ptr(), d_y.data_ptr(), k, gpu.stream))
    got, want = gpu.down(d_y).view(np.uint32), oracle.dequantize(t, blocks, 32).reshape(-1).view(np.uint32)
    nan = np.isnan(want.view(np.float32))
    assert np.array_equal(got[~nan], want[~nan]) and np.array_equal(np.isnan(got.view(np.float32)), nan)
    # empty input is a no-op
    assert pkg.kernels().mi355x_dequantize_row(t, d_b.data_ptr(), d_y.data_ptr(), 0, gpu.stream) == 0
    assert pkg.kernels().mi355x_dequantize_row(t, d_b.data_ptr(), d_y.data_ptr(), 33, gpu.stream) == -2


def test_quantize_row_q8_0_matches_activation_quantizer(pkg, oracle, gpu):
    x = rnd((64, 256), 2.0)
    x[0, :32] = 0.0
    x[1, :32] = np.arange(32) - 15.5
    d_x = gpu.up(x)
    d_q = torch.empty(x.size // 32 * 34, dtype=torch.uint8, device=gpu.dev)
    pkg.check(pkg.kernels().mi355x_quantize_row_q8_0(d_x.data_ptr(), d_q.data_ptr(), x.size, gpu.stream))
    assert np.array_equal(gpu.down(d_q).reshape(64, -1), oracle.quantize(oracle.Q8_0, x, act=True))


@pytest.mark.parametrize("wtype", ["Q5_0", "Q8_0"])
@pytest.mark.parametrize("shape", [(512, 2048, 1500), (1280, 1280, 129), (512, 130, 9), (32, 64, 200), (5120, 1280, 5), (1280, 5120, 1), (512, 1001, 3), (1280, 51866, 5), (256, 96, 8)])
def test_mul_mat_quantized(pkg, oracle, gpu, wtype, shape):
    k, m, n = shape
    if m > 20000 and wtype == "Q5_0":
        pytest.skip("one logits-sized case is enough")
    t = getattr(pkg, wtype)
    blocks = oracle.quantize(t, rnd((m, k), 0.02))
    x = rnd((n, k))
    got, name = run_mul_mat(pkg, gpu, t, blocks, x, k, m)
    assert ("gemv" in name) == (n <= 8)
    if n * m * k <= 2e9:
        want = oracle.mul_mat(t, blocks, x)
    else:                                                   # keep the scalar oracle to seconds: check a slab of rows
        sel = np.r_[0:64, m - 64:m]
        want = oracle.mul_mat(t, blocks[sel], x)
        got = got[:, sel]
    # both paths reproduce the reference's Q8_0 rounding of the activations: NMSE <= 1e-6 (GEMV: integer dot products, <= 1e-10)
    assert oracle.nmse(got, want) <= (1e-10 if n <= 8 else 1e-6)
    if n <= 8:
        # without a workspace every workgroup quantizes the activations for itself: the same integers, another summation order
        alone, _ = run_mul_mat(pkg, gpu, t, blocks, x, k, m, workspace=False)
        assert oracle.nmse(alone if n * m * k <= 2e9 else alone[:, sel], want) <= 1e-10


@pytest.mark.parametrize("shape", [(1280, 51866, 5), (1280, 2000, 8), (384, 1000, 1), (512, 51865, 3), (768, 16, 2), (1024, 333, 7), (1280, 4000, 1)])
def test_norm_mul_mat_q8_0_tiles(pkg, oracle, gpu, shape):
    # the decoder's last LayerNorm inside the launch of the logits product: the same normalized rows, Q8_0 form and logits, bit
    # for bit, as mi355x_norm_emit_q8_0 followed by mi355x_mul_mat_q8_0_tiles over the workspace
    lib = pkg.kernels()
    k, m, n = shape
    blocks = oracle.quantize(pkg.Q8_0, rnd((m, k), 0.02))
    x = rnd((n, k), 2.0, 0.3)
    w, b = rnd((k,), 0.02, 1.0), rnd((k,), 0.02)
    d_blk, d_x, d_w, d_b = gpu.up(blocks), gpu.up(x), gpu.up(w), gpu.up(b)
    size = lib.mi355x_q8_0_tiles_size(k, m)
    tiles = torch.zeros((size,), dtype=torch.uint8, device=gpu.dev)
    pkg.check(lib.mi355x_q8_0_tiles_pack(pkg.tensor(d_blk, pkg.Q8_0, ne=[k, m]), tiles.data_ptr(), gpu.stream))
    need = (n * k + n * (k // 32) * 8 + 255) // 256 * 256
    tx = pkg.tensor(d_x, pkg.F32)

    def run(fused, affine, f16):
        d_n = torch.zeros_like(d_x)
        ws = torch.zeros(need, dtype=torch.uint8, device=gpu.dev)
        d_y = torch.full((n, m), 7.0, dtype=torch.float16 if f16 else torch.float32, device=gpu.dev)
        tn, ty = pkg.tensor(d_n, pkg.F32), pkg.tensor(d_y, pkg.F16 if f16 else pkg.F32)
        pw, pb = (d_w.data_ptr(), d_b.data_ptr()) if affine else (None, None)
        fl = pkg.EPI_OUT_F16 if f16 else 0
        if fused:
            pkg.check(lib.mi355x_norm_mul_mat_q8_0_tiles(tiles.data_ptr(), k, m, tx, tn, 1e-5, pw, pb, ty, fl, ws.data_ptr(), need, gpu.stream))
        else:
            pkg.check(lib.mi355x_norm_emit_q8_0(tx, tn, 1e-5, pw, pb, ws.data_ptr(), gpu.stream))
            pkg.check(lib.mi355x_mul_mat_q8_0_tiles(tiles.data_ptr(), k, m, tn, ty, fl | pkg.MM_WS_READY, ws.data_ptr(), need, gpu.stream))
        y = gpu.down(d_y)
        return gpu.down(d_n), gpu.down(ws)[: n * k + n * (k // 32) * 8], y.view(np.uint16) if f16 else y

    for affine, f16 in ((True, False), (False, False), (True, True)):
        n1, q1, y1 = run(True, affine, f16)
        n0, q0, y0 = run(False, affine, f16)
        assert np.array_equal(n1, n0) and np.array_equal(q1, q0) and np.array_equal(y1, y0), (affine, f16)
        if affine and not f16:
            assert oracle.nmse(n1, oracle.norm(x, 1e-5) * w + b) <= 1e-10
            sel = np.r_[0:min(64, m), max(m - 64, 0):m]
            assert oracle.nmse(y1[:, sel], oracle.mul_mat(pkg.Q8_0, blocks.reshape(m, -1)[sel], n1)) <= 1e-10
    # what it does not take: another K, no workspace, rows of another length, flags of the plain product
    d_n = torch.zeros_like(d_x)
    d_y = torch.zeros((n, m), dtype=torch.float32, device=gpu.dev)
    ws = torch.zeros(need, dtype=torch.uint8, device=gpu.dev)
    tn, ty = pkg.tensor(d_n, pkg.F32), pkg.tensor(d_y, pkg.F32)
    assert lib.mi355x_norm_mul_mat_q8_0_tiles(tiles.data_ptr(), 640, m, tx, tn, 1e-5, None, None, ty, 0, ws.data_ptr(), need, gpu.stream) == -1
    assert lib.mi355x_norm_mul_mat_q8_0_tiles(tiles.data_ptr(), k, m, tx, tn, 1e-5, None, None, ty, 0, None, 0, gpu.stream) == -3
    assert lib.mi355x_norm_mul_mat_q8_0_tiles(tiles.data_ptr(), k, m, tx, tn, 1e-5, None, None, ty, pkg.MM_WS_READY, ws.data_ptr(), need, gpu.stream) == -1
    assert lib.mi355x_norm_mul_mat_q8_0_tiles(tiles.data_ptr(), k, m + 16, tx, tn, 1e-5, None, None, ty, 0, ws.data_ptr(), need, gpu.stream) == -2


@pytest.mark.parametrize("shape", [(1280, 51866, 5), (1280, 2000, 8), (384, 1000, 1), (512, 47, 3), (768, 16, 2), (1024, 333, 7)])
def test_mul_mat_q8_0_tiles(pkg, oracle, gpu, shape):
    # the matrix-core form of the few-column product: the block rows repacked 16 rows x 2 blocks at a time
    lib = pkg.kernels()
    k, m, n = shape
    blocks = oracle.quantize(pkg.Q8_0, rnd((m, k), 0.02))
    x = rnd((n, k))
    d_w, d_x = gpu.up(blocks), gpu.up(x)
    tw, tx = pkg.tensor(d_w, pkg.Q8_0, ne=[k, m]), pkg.tensor(d_x, pkg.F32)
    size = lib.mi355x_q8_0_tiles_size(k, m)
    assert size == -(-m // 16) * (k // 64) * 1088
    tiles = torch.full((size,), 0xAA, dtype=torch.uint8, device=gpu.dev)
    pkg.check(lib.mi355x_q8_0_tiles_pack(tw, tiles.data_ptr(), gpu.stream))
    # the repacked bytes: lane l of a (tile, step) holds 16 quants of row 16 tile + l % 16, block 2 step + l / 32, half (l / 16) % 2
    img = gpu.down(tiles).reshape(-(-m // 16), k // 64, 1088)
    rows = np.zeros((-(-m // 16) * 16, k // 32, 34), dtype=np.uint8)
    rows[:m] = blocks.reshape(m, k // 32, 34)
    rows = rows.reshape(-1, 16, k // 64, 2, 34)                                   # [tile][r][step][block of the pair][34]
    quants = rows[..., 2:].reshape(rows.shape[0], 16, k // 64, 2, 2, 16)           # ... [half][16]
    want_q = quants.transpose(0, 2, 3, 4, 1, 5).reshape(rows.shape[0], k // 64, 1024)   # [tile][step][g = 2 block + half][r][16]
    assert np.array_equal(img[:, :, :1024], want_q)
    want_d = rows[..., :2].transpose(0, 2, 3, 1, 4).reshape(rows.shape[0], k // 64, 64)  # [tile][step][block][r][2]
    assert np.array_equal(img[:, :, 1024:], want_d)

    need = n * k + n * (k // 32) * 8
    ws = torch.zeros((need + 255) // 256 * 256, dtype=torch.uint8, device=gpu.dev)
    d_y = torch.full((n, m), 7.0, dtype=torch.float32, device=gpu.dev)
    pkg.check(lib.mi355x_mul_mat_q8_0_tiles(tiles.data_ptr(), k, m, tx, pkg.tensor(d_y, pkg.F32), 0, ws.data_ptr(), ws.numel(), gpu.stream))
    got = gpu.down(d_y)
    sel = np.r_[0:min(64, m), max(m - 64, 0):m] if n * m * k > 2e9 else np.arange(m)
    want = oracle.mul_mat(pkg.Q8_0, blocks.reshape(m, -1)[sel], x)
    assert oracle.nmse(got[:, sel], want) <= 1e-10          # the reference's integer sums and scales; f32 order of the blocks differs
    # f16 output, over the activations already in the workspace
    d_h = torch.zeros((n, m), dtype=torch.float16, device=gpu.dev)
    d_x.zero_()
    pkg.check(lib.mi355x_mul_mat_q8_0_tiles(tiles.data_ptr(), k, m, tx, pkg.tensor(d_h, pkg.F16), pkg.EPI_OUT_F16 | pkg.MM_WS_READY, ws.data_ptr(), ws.numel(), gpu.stream))
    assert np.array_equal(gpu.down(d_h).view(np.uint16), oracle.f32_to_f16_bits(got))
    # shapes and arguments it does not take
    assert lib.mi355x_q8_0_tiles_size(96, 16) == 0
    assert lib.mi355x_mul_mat_q8_0_tiles(tiles.data_ptr(), k, m, tx, pkg.tensor(d_y, pkg.F32), 0, None, 0, gpu.stream) == -3
    assert lib.mi355x_mul_mat_q8_0_tiles(tiles.data_ptr(), 640, m, tx, pkg.tensor(d_y, pkg.F32), 0, ws.data_ptr(), ws.numel(), gpu.stream) == -1


def test_gemv_over_activations_quantized_ahead(pkg, oracle, gpu):
    # MI355X_MM_PREPARE_ONLY leaves the quantized activations in the workspace; products over them pass MI355X_MM_WS_READY
    lib = pkg.kernels()
    k, n = 1280, 5
    x = rnd((n, k))
    d_x = gpu.up(x)
    tx = pkg.tensor(d_x, pkg.F32)
    mats = [(pkg.Q8_0, 1280), (pkg.Q8_0, 640), (pkg.Q5_0, 5120)]
    ws = None
    for step, (t, m) in enumerate(mats):
        blocks = oracle.quantize(t, rnd((m, k), 0.02))
        d_w = gpu.up(blocks)
        tw = pkg.tensor(d_w, t, ne=[k, m])
        need = lib.mi355x_mul_mat_workspace_size(tw, tx)
        assert need >= n * k + n * (k // 32) * 8
        epi = pkg.Epilogue()
        if ws is None:
            ws = torch.zeros(need, dtype=torch.uint8, device=gpu.dev)
            epi.flags = pkg.MM_PREPARE_ONLY
            pkg.check(lib.mi355x_mul_mat(tw, tx, pkg.tensor(torch.empty((n, m), device=gpu.dev), pkg.F32), C.byref(epi), ws.data_ptr(), need, gpu.stream))
            image = gpu.down(ws)
            q = oracle.quantize(oracle.Q8_0, x, act=True).reshape(n, k // 32, 34)
            assert np.array_equal(image[: n * k].reshape(n, k // 32, 32), q[:, :, 2:])
            scales = image[n * k : n * k + n * (k // 32) * 4].view(np.float32).reshape(n, k // 32)
            assert np.array_equal(scales, oracle.f16_bits_to_f32(q[:, :, :2].copy().view(np.uint16)[..., 0]))
        assert need <= ws.numel()
        d_y = torch.zeros((n, m), dtype=torch.float32, device=gpu.dev)
        epi.flags = pkg.MM_WS_READY
        d_x.zero_() if step == len(mats) - 1 else None      # the last product must not look at src1 any more
        pkg.check(lib.mi355x_mul_mat(tw, tx, pkg.tensor(d_y, pkg.F32), C.byref(epi), ws.data_ptr(), need, gpu.stream))
        assert oracle.nmse(gpu.down(d_y), oracle.mul_mat(t, blocks, x)) <= 1e-10


@pytest.mark.parametrize("wtype", ["F16", "F32"])
@pytest.mark.parametrize("shape", [(1280, 1280, 300), (240, 512, 200), (37, 50, 11), (1280, 640, 1)])
def test_mul_mat_float_weights(pkg, oracle, gpu, wtype, shape):
    k, m, n = shape
    t = getattr(pkg, wtype)
    w = rnd((m, k), 0.02)
    wdata = oracle.f32_to_f16_bits(w) if t == pkg.F16 else w
    x = rnd((n, k))
    got, _ = run_mul_mat(pkg, gpu, t, wdata, x, k, m)
    assert oracle.nmse(got, oracle.mul_mat(t, wdata, x)) <= 1e-6        # f16 operands, f32 accumulation


def test_mul_mat_exact_activation_mode_is_closer_to_float64(pkg, oracle, gpu):
    k, m, n = 1280, 256, 100
    blocks = oracle.quantize(pkg.Q5_0, rnd((m, k), 0.02))
    x = rnd((n, k))
    exact = x.astype(np.float64) @ oracle.dequantize(pkg.Q5_0, blocks, k).astype(np.float64).T
    faithful, _ = run_mul_mat(pkg, gpu, pkg.Q5_0, blocks, x, k, m)
    precise, _ = run_mul_mat(pkg, gpu, pkg.Q5_0, blocks, x, k, m, flags=pkg.MM_EXACT_ACT)
    assert oracle.nmse(precise, exact) < 1e-6 < oracle.nmse(faithful, exact) < 5e-4


def test_mul_mat_epilogues(pkg, oracle, gpu):
    k, m, n = 512, 384, 150
    blocks = oracle.quantize(pkg.Q8_0, rnd((m, k), 0.02))
    for nn in (n, 5):
        x, bias, resid = rnd((nn, k)), rnd((m,), 0.5), rnd((nn, m))
        base = oracle.mul_mat(pkg.Q8_0, blocks, x)
        got, _ = run_mul_mat(pkg, gpu, pkg.Q8_0, blocks, x, k, m, flags=pkg.EPI_BIAS | pkg.EPI_GELU, bias=bias)
        assert oracle.nmse(got, oracle.gelu(base + bias)) <= 1e-5
        got, _ = run_mul_mat(pkg, gpu, pkg.Q8_0, blocks, x, k, m, flags=pkg.EPI_BIAS | pkg.EPI_RESIDUAL, bias=bias, resid=resid)
        assert oracle.nmse(got, base + bias + resid) <= 1e-6
        got, _ = run_mul_mat(pkg, gpu, pkg.Q8_0, blocks, x, k, m, flags=pkg.EPI_BIAS | pkg.EPI_SCALE, bias=bias, scale=0.35355339)
        assert oracle.nmse(got, (base + bias) * np.float32(0.35355339)) <= 1e-6
        got, _ = run_mul_mat(pkg, gpu, pkg.Q8_0, blocks, x, k, m, flags=pkg.EPI_SCALE, scale=0.35355339, out_f16=True)
        want16 = oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(base * np.float32(0.35355339)))
        assert oracle.nmse(got, want16) <= 1e-6
        colbias = rnd((nn,), 0.5)
        got, _ = run_mul_mat(pkg, gpu, pkg.Q8_0, blocks, x, k, m, flags=pkg.EPI_BIAS_COL, bias=colbias)
        assert oracle.nmse(got, base + colbias[:, None]) <= 1e-6


def test_mul_mat_gelu_epilogue_from_the_lds_table_slice(pkg, oracle, gpu):
    # On 128 x 128 tiles (the FFN-up shape) the GELU epilogue looks its values up in the part of the f16 table kept in LDS
    # (|x| < 8) and goes to the table in global memory for anything larger: both routes, against the standalone GELU kernel
    # on the product without the epilogue — the same table, so the same bits.
    lib = pkg.kernels()
    k, m, n = 256, 2560, 1500
    blocks = oracle.quantize(pkg.Q8_0, rnd((m, k), 0.02))
    x = rnd((n, k))
    bias = rnd((m,), 2.0)
    bias[::97] = 40.0 * np.sign(bias[::97])                 # a few columns far outside the slice (|x| >= 8, and beyond the clamps at 10)
    bias[5::89] = 8.5
    plain, name = run_mul_mat(pkg, gpu, pkg.Q8_0, blocks, x, k, m, flags=pkg.EPI_BIAS, bias=bias)
    got, _ = run_mul_mat(pkg, gpu, pkg.Q8_0, blocks, x, k, m, flags=pkg.EPI_BIAS | pkg.EPI_GELU, bias=bias)
    assert "gemm" in name
    d_p = gpu.up(plain)
    d_g = torch.empty_like(d_p)
    pkg.check(lib.mi355x_gelu(pkg.tensor(d_p, pkg.F32), pkg.tensor(d_g, pkg.F32), gpu.stream))
    want = gpu.down(d_g)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert (np.abs(plain) >= 8).sum() > 1000 and (np.abs(plain) < 8).sum() > 1000
    assert oracle.nmse(got[:64], oracle.gelu(plain[:64])) <= 1e-7


@pytest.mark.parametrize("k,m,n", [(256, 320, 150), (256, 5120, 1500), (128, 2080, 2950)])
def test_mul_mat_epilogue_emits_the_next_products_activation_image(pkg, oracle, gpu, k, m, n):
    # MI355X_EPI_EMIT_F16: besides dst (here with bias and GELU, the FFN's first matrix), its rows rounded to Q8_0 as f16(q * d).
    # The second case has the large-v3 FFN's width and rows: the 128 x 128 tiles whose operands go straight into LDS, and whose
    # patches this epilogue forms transposed (a lane owns half a Q8_0 block); the third ends in tiles that dst covers in part
    # along both axes (32 of 128 columns, 6 of 128 rows).
    lib = pkg.kernels()
    blocks = oracle.quantize(pkg.Q5_0, rnd((m, k), 0.05))
    x, bias = rnd((n, k)), rnd((m,), 0.5)
    d_w, d_x, d_b = gpu.up(blocks), gpu.up(x), gpu.up(bias)
    d_y = torch.zeros((n, m), dtype=torch.float32, device=gpu.dev)
    d_h = torch.zeros((n, m), dtype=torch.float16, device=gpu.dev)
    tw, tx, ty = pkg.tensor(d_w, pkg.Q5_0, ne=[k, m]), pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32)
    need = lib.mi355x_mul_mat_workspace_size(tw, tx)
    ws = torch.empty(need, dtype=torch.uint8, device=gpu.dev)
    epi = pkg.Epilogue()
    epi.flags, epi.scale, epi.bias, epi.image = pkg.EPI_BIAS | pkg.EPI_GELU | pkg.EPI_EMIT_F16, 1.0, d_b.data_ptr(), d_h.data_ptr()
    pkg.check(lib.mi355x_mul_mat(tw, tx, ty, C.byref(epi), ws.data_ptr(), need, gpu.stream))
    y = gpu.down(d_y)
    assert oracle.nmse(y, oracle.gelu(oracle.mul_mat(pkg.Q5_0, blocks, x) + bias)) <= 1e-5
    image = oracle.dequantize(oracle.Q8_0, oracle.quantize(oracle.Q8_0, y, act=True), m).reshape(n, m)
    assert np.array_equal(gpu.down(d_h, np.uint16), oracle.f32_to_f16_bits(image))
    # MI355X_EPI_IMAGE_ONLY: the same image, dst untouched (its data pointer may be NULL); not without the image
    d_h2 = torch.zeros((n, m), dtype=torch.float16, device=gpu.dev)
    epi.flags, epi.image = pkg.EPI_BIAS | pkg.EPI_GELU | pkg.EPI_EMIT_F16 | pkg.EPI_IMAGE_ONLY, d_h2.data_ptr()
    d_y.fill_(7.0)
    pkg.check(lib.mi355x_mul_mat(tw, tx, ty, C.byref(epi), ws.data_ptr(), need, gpu.stream))
    assert np.array_equal(gpu.down(d_h2, np.uint16), gpu.down(d_h, np.uint16)) and np.all(gpu.down(d_y) == 7.0)
    t_null = pkg.tensor(d_y, pkg.F32); t_null.data = None
    d_h2.zero_()
    pkg.check(lib.mi355x_mul_mat(tw, tx, t_null, C.byref(epi), ws.data_ptr(), need, gpu.stream))
    assert np.array_equal(gpu.down(d_h2, np.uint16), gpu.down(d_h, np.uint16))
    epi.flags = pkg.EPI_BIAS | pkg.EPI_IMAGE_ONLY
    assert lib.mi355x_mul_mat(tw, tx, ty, C.byref(epi), ws.data_ptr(), need, gpu.stream) == -2
    # the epilogue's other terms in the same launch: scale and residual, no GELU (and dst as f16 is not an option with the image)
    res = rnd((n, m))
    d_r = gpu.up(res)
    epi.flags, epi.scale, epi.residual, epi.image = pkg.EPI_BIAS | pkg.EPI_SCALE | pkg.EPI_RESIDUAL | pkg.EPI_EMIT_F16, 0.75, d_r.data_ptr(), d_h2.data_ptr()
    pkg.check(lib.mi355x_mul_mat(tw, tx, ty, C.byref(epi), ws.data_ptr(), need, gpu.stream))
    y = gpu.down(d_y)
    assert oracle.nmse(y, (oracle.mul_mat(pkg.Q5_0, blocks, x) + bias) * np.float32(0.75) + res) <= 1e-5
    image = oracle.dequantize(oracle.Q8_0, oracle.quantize(oracle.Q8_0, y, act=True), m).reshape(n, m)
    assert np.array_equal(gpu.down(d_h2, np.uint16), oracle.f32_to_f16_bits(image))
    epi.flags |= pkg.EPI_OUT_F16
    assert lib.mi355x_mul_mat(tw, tx, ty, C.byref(epi), ws.data_ptr(), need, gpu.stream) == -2
    epi.flags, epi.scale, epi.residual, epi.image = pkg.EPI_BIAS | pkg.EPI_GELU | pkg.EPI_EMIT_F16, 1.0, None, d_h.data_ptr()
    # the GEMV path has no such epilogue
    d_x5 = gpu.up(x[:5])
    d_y5 = torch.zeros((5, m), dtype=torch.float32, device=gpu.dev)
    assert lib.mi355x_mul_mat(tw, pkg.tensor(d_x5, pkg.F32), pkg.tensor(d_y5, pkg.F32), C.byref(epi), ws.data_ptr(), need, gpu.stream) == -1


@pytest.mark.parametrize("k,m,n", [(512, 384, 200), (1280, 1280, 1500)])
def test_mul_mat_group_equals_single_calls(pkg, oracle, gpu, k, m, n):
    # three products over the same activations (the shape of a layer's Q, K, V projections) as one launch: same bits as
    # three calls, each with its own epilogue and destination type.  The second case is a large-v3 encoder layer's, which
    # the grouped form runs on 128 x 192 tiles (one workgroup to a CU) with a partial last tile column.
    lib = pkg.kernels()
    x = rnd((n, k))
    d_x = gpu.up(x)
    tx = pkg.tensor(d_x, pkg.F32)
    images, singles, grouped, items, keep = [], [], [], (pkg.MulMatItem * 3)(), []
    specs = [(pkg.EPI_BIAS, torch.float32), (0, torch.float32), (pkg.EPI_BIAS | pkg.EPI_OUT_F16, torch.float16)]
    for i, (flags, dt) in enumerate(specs):
        blocks = oracle.quantize(pkg.Q5_0, rnd((m, k), 0.02))
        d_b = gpu.up(blocks)
        img = torch.empty((m, k), dtype=torch.float16, device=gpu.dev)
        pkg.check(lib.mi355x_dequantize_row_f16(pkg.Q5_0, d_b.data_ptr(), img.data_ptr(), m * k, gpu.stream))
        bias = gpu.up(rnd((m,), 0.5))
        epi = pkg.Epilogue(); epi.flags, epi.scale, epi.bias = flags, 1.0, bias.data_ptr()
        tw = pkg.tensor(img, pkg.F16)
        y1, y2 = torch.zeros((n, m), dtype=dt, device=gpu.dev), torch.zeros((n, m), dtype=dt, device=gpu.dev)
        t1, t2 = pkg.tensor(y1, pkg.F16 if dt == torch.float16 else pkg.F32), pkg.tensor(y2, pkg.F16 if dt == torch.float16 else pkg.F32)
        keep += [d_b, img, bias, epi, tw, t1, t2]
        images.append(tw); singles.append((y1, t1, epi)); grouped.append(y2)
        items[i].src0, items[i].dst, items[i].epi = C.pointer(tw), C.pointer(t2), C.pointer(epi)
    need = lib.mi355x_mul_mat_workspace_size(images[0], tx)
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device=gpu.dev)
    for tw, (y1, t1, epi) in zip(images, singles):
        one = pkg.Epilogue(); one.flags, one.scale, one.bias = epi.flags | pkg.MM_ACT_Q8_0, 1.0, epi.bias
        pkg.check(lib.mi355x_mul_mat(tw, tx, t1, C.byref(one), ws.data_ptr(), need, gpu.stream))
    rc = lib.mi355x_mul_mat_group(items, 3, tx, pkg.MM_ACT_Q8_0, ws.data_ptr(), need, gpu.stream)
    pkg.check(rc, "mul_mat_group")
    for (y1, _, _), y2 in zip(singles, grouped):
        assert torch.equal(y1, y2)
    assert float(grouped[1].abs().sum()) > 0
    # shapes outside its one purpose are declined, not mis-computed: K = 96 is no multiple of 256
    small = torch.zeros((m, 96), dtype=torch.float16, device=gpu.dev)
    xs = torch.zeros((n, 96), dtype=torch.float32, device=gpu.dev)
    it = (pkg.MulMatItem * 1)()
    tws, tds = pkg.tensor(small, pkg.F16), pkg.tensor(grouped[1], pkg.F32)
    it[0].src0, it[0].dst, it[0].epi = C.pointer(tws), C.pointer(tds), None
    assert lib.mi355x_mul_mat_group(it, 1, pkg.tensor(xs, pkg.F32), 0, ws.data_ptr(), need, gpu.stream) == -1


@pytest.mark.parametrize("wtype,n", [("Q8_0", 5), ("Q5_0", 1), ("Q8_0", 8)])
def test_mul_mat_group_few_columns(pkg, oracle, gpu, wtype, n):
    # a decode step's Q, K and V in one launch: the same results as single calls (same kernel body, same order of sums)
    lib = pkg.kernels()
    t = getattr(pkg, wtype)
    k, m = 1280, 1280
    x = rnd((n, k))
    d_x = gpu.up(x)
    tx = pkg.tensor(d_x, pkg.F32)
    mats = [oracle.quantize(t, rnd((m, k), 0.02)) for _ in range(3)]
    d_w = [gpu.up(b) for b in mats]
    tws = [pkg.tensor(w, t, ne=[k, m]) for w in d_w]
    bias = rnd((m,), 0.5)
    d_b = gpu.up(bias)
    need = lib.mi355x_mul_mat_workspace_size(tws[0], tx)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=gpu.dev)
    outs = [torch.zeros((n, m), dtype=torch.float32, device=gpu.dev), torch.zeros((n, m), dtype=torch.float16, device=gpu.dev),
            torch.zeros((n, m), dtype=torch.float32, device=gpu.dev)]
    tds = [pkg.tensor(outs[0], pkg.F32), pkg.tensor(outs[1], pkg.F16), pkg.tensor(outs[2], pkg.F32)]
    epis = [pkg.Epilogue() for _ in range(3)]
    epis[0].flags, epis[0].scale, epis[0].bias = pkg.EPI_BIAS | pkg.EPI_SCALE, 0.125, d_b.data_ptr()
    epis[1].flags, epis[1].scale = pkg.EPI_OUT_F16, 1.0
    epis[2].flags, epis[2].scale, epis[2].bias = pkg.EPI_BIAS, 1.0, d_b.data_ptr()
    items = (pkg.MulMatItem * 3)()
    for i in range(3):
        items[i].src0, items[i].dst, items[i].epi = C.pointer(tws[i]), C.pointer(tds[i]), C.pointer(epis[i])
    pkg.check(lib.mi355x_mul_mat_group(items, 3, tx, 0, ws.data_ptr(), need, gpu.stream))
    got = [gpu.down(o).astype(np.float32) for o in outs]
    for i in range(3):
        single = torch.zeros_like(outs[i])
        pkg.check(lib.mi355x_mul_mat(tws[i], tx, pkg.tensor(single, pkg.F16 if i == 1 else pkg.F32), C.byref(epis[i]), ws.data_ptr(), need, gpu.stream))
        assert np.array_equal(got[i], gpu.down(single).astype(np.float32))
    base = [oracle.mul_mat(t, b, x) for b in mats]
    assert oracle.nmse(got[0], (base[0] + bias) * np.float32(0.125)) <= 1e-10
    assert oracle.nmse(got[1], oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(base[1]))) <= 1e-7     # an f32 ulp can move an f16 rounding
    assert oracle.nmse(got[2], base[2] + bias) <= 1e-10
    # without the workspace the grouped form has nothing to read the activations from
    assert lib.mi355x_mul_mat_group(items, 3, tx, 0, None, 0, gpu.stream) == -3


@pytest.mark.parametrize("wtype,n,k,m,count", [("Q8_0", 5, 1280, 1280, 3), ("Q8_0", 5, 1280, 5120, 1), ("Q5_0", 1, 512, 384, 2), ("Q8_0", 8, 768, 51866, 1)])
def test_norm_mul_mat_group(pkg, oracle, gpu, wtype, n, k, m, count):
    # LayerNorm + affine and the few-column products over its rows in one launch: the same rows, the same Q8_0 form and the
    # same products as mi355x_norm_emit_q8_0 followed by mi355x_mul_mat_group
    lib = pkg.kernels()
    t = getattr(pkg, wtype)
    x = rnd((n, k), 2.0, 0.3)
    w, b = rnd((k,), 0.02, 1.0), rnd((k,), 0.02)
    d_x, d_w, d_b = gpu.up(x), gpu.up(w), gpu.up(b)
    mats = [oracle.quantize(t, rnd((m, k), 0.02)) for _ in range(count)]
    d_m = [gpu.up(q) for q in mats]
    tws = [pkg.tensor(q, t, ne=[k, m]) for q in d_m]
    bias = rnd((m,), 0.5)
    d_bias = gpu.up(bias)
    tx = pkg.tensor(d_x, pkg.F32)
    need = lib.mi355x_mul_mat_workspace_size(tws[0], tx)
    assert need > 0

    def run(fused):
        d_y = torch.zeros_like(d_x)
        ws = torch.zeros(need, dtype=torch.uint8, device=gpu.dev)
        outs = [torch.zeros((n, m), dtype=torch.float32, device=gpu.dev) for _ in range(count)]
        tds = [pkg.tensor(o, pkg.F32) for o in outs]
        epis = [pkg.Epilogue() for _ in range(count)]
        for e in epis:
            e.flags, e.scale, e.bias = pkg.EPI_BIAS, 1.0, d_bias.data_ptr()
        items = (pkg.MulMatItem * count)()
        for i in range(count):
            items[i].src0, items[i].dst, items[i].epi = C.pointer(tws[i]), C.pointer(tds[i]), C.pointer(epis[i])
        ty = pkg.tensor(d_y, pkg.F32)
        if fused:
            pkg.check(lib.mi355x_norm_mul_mat_group(tx, ty, 1e-5, d_w.data_ptr(), d_b.data_ptr(), items, count, ws.data_ptr(), need, gpu.stream))
        else:
            pkg.check(lib.mi355x_norm_emit_q8_0(tx, ty, 1e-5, d_w.data_ptr(), d_b.data_ptr(), ws.data_ptr(), gpu.stream))
            pkg.check(lib.mi355x_mul_mat_group(items, count, ty, pkg.MM_WS_READY, ws.data_ptr(), need, gpu.stream))
        return gpu.down(d_y), gpu.down(ws)[: n * k + n * (k // 32) * 8], [gpu.down(o) for o in outs]

    y1, q1, o1 = run(True)
    y0, q0, o0 = run(False)
    assert np.array_equal(y1, y0) and np.array_equal(q1, q0)
    for a, bb in zip(o1, o0):
        assert np.array_equal(a, bb)
    assert oracle.nmse(y1, oracle.norm(x, 1e-5) * w + b) <= 1e-10
    sel = np.r_[0:32, m - 32:m]
    assert oracle.nmse(o1[0][:, sel], oracle.mul_mat(t, mats[0][sel], y1) + bias[sel]) <= 1e-10
    # rows too long for the register-resident LayerNorm say so
    if k == 1280:
        long = torch.zeros((n, 4096), dtype=torch.float32, device=gpu.dev)
        tl = pkg.tensor(long, pkg.F32)
        assert lib.mi355x_norm_mul_mat_group(tl, tl, 1e-5, None, None, (pkg.MulMatItem * 1)(), 1, None, 0, gpu.stream) in (-1, -2)


@pytest.mark.parametrize("wtype,ttype,n,k,m,count", [("Q8_0", "Q8_0", 5, 1280, 1280, 3), ("Q5_0", "F16", 3, 512, 512, 3), ("Q8_0", "F16", 8, 384, 384, 3),
                                                     ("Q5_0", "Q8_0", 1, 1280, 1280, 3), ("Q8_0", "Q8_0", 2, 768, 768, 1), ("Q5_0", "Q5_0", 5, 1280, 1280, 3),
                                                     ("Q5_0", "Q5_0", 7, 512, 512, 3)])
def test_embed_norm_mul_mat_group(pkg, oracle, gpu, wtype, ttype, n, k, m, count):
    # the token + positional embedding of a decode step made inside the launch that normalizes it and multiplies: the same
    # embedding rows, normalized rows, Q8_0 form and products, bit for bit, as mi355x_get_rows_add followed by
    # mi355x_norm_mul_mat_group
    lib = pkg.kernels()
    t, tt = getattr(pkg, wtype), getattr(pkg, ttype)
    n_vocab, n_ctx = 300, 48
    table = rnd((n_vocab, k), 0.05)
    tok = oracle.quantize(tt, table) if tt != pkg.F16 else oracle.f32_to_f16_bits(table)
    pos = rnd((n_ctx, k), 0.05)
    w, b = rnd((k,), 0.02, 1.0), rnd((k,), 0.02)
    d_tok, d_pos, d_w, d_b = gpu.up(tok), gpu.up(pos), gpu.up(w), gpu.up(b)
    t_tok, t_pos = pkg.tensor(d_tok, tt, ne=[k, n_vocab]), pkg.tensor(d_pos, pkg.F32)
    mats = [oracle.quantize(t, rnd((m, k), 0.02)) for _ in range(count)]
    d_m = [gpu.up(q) for q in mats]
    tws = [pkg.tensor(q, t, ne=[k, m]) for q in d_m]
    need = lib.mi355x_mul_mat_workspace_size(tws[0], pkg.tensor(torch.zeros((n, k), dtype=torch.float32, device=gpu.dev), pkg.F32))
    assert need > 0

    def run(fused, ids, pids):
        d_i, d_pi = gpu.up(ids), gpu.up(pids)
        t_i, t_pi = pkg.tensor(d_i, pkg.I32), pkg.tensor(d_pi, pkg.I32)
        d_x = torch.full((n, k), 7.0, dtype=torch.float32, device=gpu.dev)
        d_y = torch.zeros_like(d_x)
        ws = torch.zeros(need, dtype=torch.uint8, device=gpu.dev)
        outs = [torch.zeros((n, m), dtype=torch.float32, device=gpu.dev) for _ in range(count)]
        tds = [pkg.tensor(o, pkg.F32) for o in outs]
        items = (pkg.MulMatItem * count)()
        for i in range(count):
            items[i].src0, items[i].dst, items[i].epi = C.pointer(tws[i]), C.pointer(tds[i]), None
        tx, ty = pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32)
        if fused:
            pkg.check(lib.mi355x_embed_norm_mul_mat_group(t_tok, t_i, t_pos, t_pi, tx, ty, 1e-5, d_w.data_ptr(), d_b.data_ptr(), items, count, ws.data_ptr(), need, gpu.stream))
        else:
            pkg.check(lib.mi355x_get_rows_add(t_tok, t_i, t_pos, t_pi, tx, gpu.stream))
            pkg.check(lib.mi355x_norm_mul_mat_group(tx, ty, 1e-5, d_w.data_ptr(), d_b.data_ptr(), items, count, ws.data_ptr(), need, gpu.stream))
        return gpu.down(d_x), gpu.down(d_y), gpu.down(ws)[: n * k + n * (k // 32) * 8], [gpu.down(o) for o in outs]

    ids = np.array([5, 299, 0, 5, 17, 123, 1, 298], dtype=np.int32)[:n]
    pids = np.array([7, 8, 47, 0, 7, 9, 10, 11], dtype=np.int32)[:n]
    x1, y1, q1, o1 = run(True, ids, pids)
    x0, y0, q0, o0 = run(False, ids, pids)
    if tt != pkg.F16:
        assert np.array_equal(x0, oracle.binary(0, oracle.get_rows(tt, tok, ids, k), pos[pids]))
    else:
        assert np.array_equal(x0, oracle.f16_bits_to_f32(tok[ids]) + pos[pids])
    assert np.array_equal(x1, x0) and np.array_equal(y1, y0) and np.array_equal(q1, q0)
    for a, bb in zip(o1, o0):
        assert np.array_equal(a, bb)
    # an index outside its table: a NaN row, as from the launch of its own, and the rows beside it untouched by that
    if n >= 3:
        bad, pbad = ids.copy(), pids.copy()
        bad[1], pbad[2] = n_vocab, -1
        x1, y1, _, o1 = run(True, bad, pbad)
        x0, y0, _, o0 = run(False, bad, pbad)
        assert np.isnan(x1[[1, 2]]).all() and np.isnan(y1[[1, 2]]).all()
        keep = [r for r in range(n) if r not in (1, 2)]
        assert np.array_equal(x1[keep], x0[keep]) and np.array_equal(y1[keep], y0[keep]) and np.array_equal(o1[0][keep], o0[0][keep])
    # index vectors of another length, a table of another width, a token table of a type the launch does not read
    d_i, d_pi = gpu.up(ids), gpu.up(pids)
    d_x = torch.zeros((n, k), dtype=torch.float32, device=gpu.dev)
    tx = pkg.tensor(d_x, pkg.F32)
    items = (pkg.MulMatItem * 1)()
    out = torch.zeros((n, m), dtype=torch.float32, device=gpu.dev)
    td = pkg.tensor(out, pkg.F32)
    items[0].src0, items[0].dst, items[0].epi = C.pointer(tws[0]), C.pointer(td), None
    ws = torch.zeros(need, dtype=torch.uint8, device=gpu.dev)
    args = (1e-5, d_w.data_ptr(), d_b.data_ptr(), items, 1, ws.data_ptr(), need, gpu.stream)
    if n > 1:
        assert lib.mi355x_embed_norm_mul_mat_group(t_tok, pkg.tensor(d_i[: n - 1], pkg.I32), t_pos, pkg.tensor(d_pi, pkg.I32), tx, tx, *args) == -1
    assert lib.mi355x_embed_norm_mul_mat_group(t_tok, pkg.tensor(d_i, pkg.I32), pkg.tensor(d_pos[:, : k - 32], pkg.F32), pkg.tensor(d_pi, pkg.I32), tx, tx, *args) == -2
    assert lib.mi355x_embed_norm_mul_mat_group(pkg.tensor(d_pos, pkg.F32), pkg.tensor(d_i, pkg.I32), t_pos, pkg.tensor(d_pi, pkg.I32), tx, tx, *args) == -1
    assert lib.mi355x_embed_norm_mul_mat_group(None, pkg.tensor(d_i, pkg.I32), t_pos, pkg.tensor(d_pi, pkg.I32), tx, tx, *args) == -2


@pytest.mark.parametrize("wtype,n,k,m", [("Q8_0", 5, 1280, 5120), ("Q5_0", 3, 512, 384), ("Q8_0", 8, 384, 1536), ("Q8_0", 1, 1280, 5120)])
def test_few_column_product_emits_its_result_as_q8_0(pkg, oracle, gpu, wtype, n, k, m):
    # MI355X_EPI_EMIT_Q8_0: a decode step's FFN-up product (bias + GELU) leaves its rows quantized for FFN-down, in the layout
    # the quantization pass of that product would write (quants | f16-rounded scales as f32 | block sums): through
    # mi355x_mul_mat, mi355x_mul_mat_group with one product and mi355x_norm_mul_mat_group — the same bytes from all three
    lib = pkg.kernels()
    t = getattr(pkg, wtype)
    x = rnd((n, k), 1.0)
    blocks = oracle.quantize(t, rnd((m, k), 0.05))
    bias = rnd((m,), 0.5)
    d_x, d_w, d_b = gpu.up(x), gpu.up(blocks), gpu.up(bias)
    tw, tx = pkg.tensor(d_w, t, ne=[k, m]), pkg.tensor(d_x, pkg.F32)
    need = lib.mi355x_mul_mat_workspace_size(tw, tx)
    img_bytes = n * m + n * (m // 32) * 8

    def layout(image, y):
        q = oracle.quantize(oracle.Q8_0, y, act=True).reshape(n, m // 32, 34)
        assert np.array_equal(image[: n * m].reshape(n, m // 32, 32), q[:, :, 2:])
        d = image[n * m: n * m + n * (m // 32) * 4].view(np.float32).reshape(n, m // 32)
        assert np.array_equal(oracle.f32_to_f16_bits(d), q[:, :, :2].copy().view(np.uint16).reshape(n, m // 32))
        sums = image[n * m + n * (m // 32) * 4: img_bytes].view(np.int32).reshape(n, m // 32)
        assert np.array_equal(sums, q[:, :, 2:].view(np.int8).astype(np.int32).sum(axis=2))

    def run(how):
        d_y = torch.zeros((n, m), dtype=torch.float32, device=gpu.dev)
        d_i = torch.zeros(img_bytes, dtype=torch.uint8, device=gpu.dev)
        ws = torch.zeros(need, dtype=torch.uint8, device=gpu.dev)
        epi = pkg.Epilogue()
        epi.flags, epi.scale, epi.bias, epi.image = pkg.EPI_BIAS | pkg.EPI_GELU | pkg.EPI_EMIT_Q8_0, 1.0, d_b.data_ptr(), d_i.data_ptr()
        ty = pkg.tensor(d_y, pkg.F32)
        if how == "single":
            pkg.check(lib.mi355x_mul_mat(tw, tx, ty, C.byref(epi), ws.data_ptr(), need, gpu.stream))
        else:
            items = (pkg.MulMatItem * 1)()
            items[0].src0, items[0].dst, items[0].epi = C.pointer(tw), C.pointer(ty), C.pointer(epi)
            if how == "group":
                pkg.check(lib.mi355x_mul_mat_group(items, 1, tx, 0, ws.data_ptr(), need, gpu.stream))
            else:                                      # behind a LayerNorm without affine vectors, normalized rows written in place of x
                d_n = torch.zeros_like(d_x)
                pkg.check(lib.mi355x_norm_mul_mat_group(tx, pkg.tensor(d_n, pkg.F32), 1e-5, None, None, items, 1, ws.data_ptr(), need, gpu.stream))
                return gpu.down(d_y), gpu.down(d_i), gpu.down(d_n)
        return gpu.down(d_y), gpu.down(d_i)

    y, image = run("single")
    assert oracle.nmse(y, oracle.gelu(oracle.mul_mat(t, blocks, x) + bias)) <= 1e-9
    layout(image, y)
    y2, image2 = run("group")
    assert np.array_equal(y2, y) and np.array_equal(image2, image)
    y3, image3, rows = run("norm")
    assert oracle.nmse(rows, oracle.norm(x, 1e-5)) <= 1e-10
    # (a sum that lands on the other side of an f16 boundary moves its GELU table entry by one f16 step: 1e-9, not 1e-10)
    assert oracle.nmse(y3, oracle.gelu(oracle.mul_mat(t, blocks, rows) + bias)) <= 1e-9
    layout(image3, y3)
    # not for more than one product per launch, not for many columns, not without a workspace
    epi = pkg.Epilogue(); epi.flags, epi.image = pkg.EPI_EMIT_Q8_0, d_x.data_ptr()
    d_y = torch.zeros((n, m), dtype=torch.float32, device=gpu.dev)
    ty = pkg.tensor(d_y, pkg.F32)
    assert lib.mi355x_mul_mat(tw, tx, ty, C.byref(epi), None, 0, gpu.stream) == -1
    items = (pkg.MulMatItem * 2)()
    for i in range(2):
        items[i].src0, items[i].dst, items[i].epi = C.pointer(tw), C.pointer(ty), C.pointer(epi)
    ws = torch.zeros(need, dtype=torch.uint8, device=gpu.dev)
    assert lib.mi355x_mul_mat_group(items, 2, tx, 0, ws.data_ptr(), need, gpu.stream) == -1


def test_mul_mat_rejects_bad_arguments(pkg, gpu):
    lib = pkg.kernels()
    d_w = torch.zeros(22 * 4, dtype=torch.uint8, device=gpu.dev)
    d_x = torch.zeros((3, 64), dtype=torch.float32, device=gpu.dev)
    d_y = torch.zeros((3, 2), dtype=torch.float32, device=gpu.dev)
    tw, tx, ty = pkg.tensor(d_w, pkg.Q5_0, ne=[64, 2]), pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32)
    assert lib.mi355x_mul_mat(None, tx, ty, None, None, 0, gpu.stream) == -2
    bad = pkg.tensor(d_y, pkg.F32, ne=[3, 3])
    assert lib.mi355x_mul_mat(tw, tx, bad, None, None, 0, gpu.stream) == -2           # dst shape does not match
    empty = pkg.tensor(d_x, pkg.F32, ne=[64, 0])
    empty_y = pkg.tensor(d_y, pkg.F32, ne=[2, 0])
    assert lib.mi355x_mul_mat(tw, empty, empty_y, None, None, 0, gpu.stream) == 0     # zero columns: nothing to do
    d_x2 = torch.zeros((40, 64), dtype=torch.float32, device=gpu.dev)
    d_y2 = torch.zeros((40, 2), dtype=torch.float32, device=gpu.dev)
    assert lib.mi355x_mul_mat(tw, pkg.tensor(d_x2, pkg.F32), pkg.tensor(d_y2, pkg.F32), None, None, 0, gpu.stream) == -3   # GEMM needs its workspace


# ------------------------------------------------------------------------------------------------------------------

def _attention_inputs(oracle, H, N, KV, flat=False, pad_from=None):
    q = rnd((H, N, 64), 0.05 if flat else 1.0)
    k, v = rnd((H, KV, 64)), rnd((H, KV, 64), 0.3, 1.0 if flat else 0.0)
    if pad_from is not None:
        k[:, pad_from:] = 0.0
        v[:, pad_from:] = 0.0
    return q, oracle.f32_to_f16_bits(k), oracle.f32_to_f16_bits(v)


def run_fa(pkg, gpu, q, kb, vb, mask, scale, mode):
    H, N, D = q.shape
    d_q, d_k, d_v = gpu.up(q), gpu.up(kb), gpu.up(vb)
    d_m = gpu.up(mask) if mask is not None else None
    d_o = torch.empty((N, H, D), dtype=torch.float32, device=gpu.dev)
    tq, tk = pkg.tensor(d_q, pkg.F32), pkg.tensor(d_k, pkg.F16)
    pkg.check(pkg.kernels().mi355x_flash_attn_ext(tq, tk, pkg.tensor(d_v, pkg.F16), pkg.tensor(d_m, pkg.F16) if d_m is not None else None,
                                                   pkg.tensor(d_o, pkg.F32), scale, mode, None, 0, gpu.stream), "flash_attn_ext")
    return gpu.down(d_o), pkg.kernels().mi355x_flash_attn_ext_kernel_name(tq, tk, mode).decode()


@pytest.mark.parametrize("case", [
    dict(H=2, N=70, KV=100), dict(H=3, N=200, KV=1536, flat=True, pad_from=1500), dict(H=20, N=5, KV=1536, flat=True, pad_from=1500),
    dict(H=4, N=1, KV=1), dict(H=4, N=5, KV=37, mask="beam"), dict(H=2, N=3, KV=200, mask="causal"), dict(H=2, N=100, KV=100, mask="causal"),
    dict(H=2, N=8, KV=448, mask="beam"), dict(H=2, N=9, KV=63),
    # the few-query kernel's stages of 192 keys: exactly one, one key into the second, and far more keys than it ever staged at once
    dict(H=2, N=1, KV=192), dict(H=2, N=4, KV=193, mask="beam"), dict(H=1, N=2, KV=7500)])
def test_flash_attn_reference_faithful(pkg, oracle, gpu, case):
    H, N, KV = case["H"], case["N"], case["KV"]
    q, kb, vb = _attention_inputs(oracle, H, N, KV, case.get("flat", False), case.get("pad_from"))
    mask = None
    if "mask" in case:
        m = np.full((-(-N // 64) * 64, KV), -np.inf, dtype=np.float32)
        for r in range(N):
            if case["mask"] == "causal":
                m[r, : KV - N + r + 1] = 0.0
            else:
                m[r, : (KV + 1) // 2] = 0.0
                m[r, [c for c in range(KV) if c % N == r]] = 0.0
        mask = oracle.f32_to_f16_bits(m)
    got, name = run_fa(pkg, gpu, q, kb, vb, mask, 0.125, pkg.FA_F16_SEQ)
    assert name == ("flash_attn.seq_row" if N <= 8 else "flash_attn.seq_tile")
    want = oracle.flash_attn_ext(q, kb, vb, None if mask is None else mask[:N], 0.125)
    assert oracle.nmse(got, want) <= 1e-6      # same key order, same f16 accumulator: only exp() and dot-product ulps differ


@pytest.mark.parametrize("case", [
    dict(H=2, N=70, KV=100), dict(H=3, N=200, KV=1536, flat=True, pad_from=1500), dict(H=2, N=100, KV=100, mask="causal"),
    dict(H=2, N=9, KV=63), dict(H=2, N=130, KV=448, mask="causal"), dict(H=2, N=64, KV=1500, flat=True),
    # masked keys in front of a row's first real key (the running maximum starts at a finite number, not at -inf)
    dict(H=2, N=70, KV=300, mask="late"), dict(H=2, N=5, KV=300, mask="late"),
    # at most 8 queries: the few-query kernel of the packed form (stages of 192 keys: one, one key into the second, many)
    dict(H=20, N=5, KV=1536, flat=True, pad_from=1500), dict(H=4, N=1, KV=1), dict(H=4, N=5, KV=37, mask="beam"), dict(H=2, N=3, KV=200, mask="causal"),
    dict(H=2, N=8, KV=448, mask="beam"), dict(H=2, N=1, KV=192), dict(H=2, N=4, KV=193, mask="beam"), dict(H=1, N=2, KV=7500), dict(H=3, N=5, KV=583, mask="beam")])
def test_flash_attn_packed_f16_chain(pkg, oracle, gpu, case):
    # MI355X_FA_F16_PK: the same key order and f16 accumulator, the step as one fused f16 multiply-add on the factor rounded
    # to f16 (the reference's arithmetic where it has f16 vector units).  Checked against the pinned restatement of the x86
    # sequence: a step of the two forms differs by the factor's rounding and by one rounding in place of two, which leaves
    # the results within 1e-5 NMSE of each other, and both equally far (several 1e-3 on flat attention) from an f64 evaluation.
    H, N, KV = case["H"], case["N"], case["KV"]
    q, kb, vb = _attention_inputs(oracle, H, N, KV, case.get("flat", False), case.get("pad_from"))
    mask = None
    if "mask" in case:
        m = np.full((-(-N // 64) * 64, KV), -np.inf, dtype=np.float32)
        for r in range(N):
            if case["mask"] == "causal":
                m[r, : KV - N + r + 1] = 0.0
            elif case["mask"] == "late":       # a row's first keys are masked (a whole tile of 64 and more for some rows), and every seventh after
                m[r, (r * 5) % 97 + 1:] = 0.0
                m[r, (r * 5) % 97 + 3::7] = -np.inf
            else:
                m[r, : (KV + 1) // 2] = 0.0
                m[r, [c for c in range(KV) if c % N == r]] = 0.0
        mask = oracle.f32_to_f16_bits(m)
    got, name = run_fa(pkg, gpu, q, kb, vb, mask, 0.125, pkg.FA_F16_PK)
    assert name == ("flash_attn.seq_row_pk" if N <= 8 else "flash_attn.seq_tile_pk")
    want = oracle.flash_attn_ext(q, kb, vb, None if mask is None else mask[:N], 0.125)
    seq, _ = run_fa(pkg, gpu, q, kb, vb, mask, 0.125, pkg.FA_F16_SEQ)
    exact = _attention_float64(oracle, q, kb, vb, None if mask is None else mask, 0.125)
    print(f"packed chain {case}: vs oracle {oracle.nmse(got, want):.3e}, x86 form vs oracle {oracle.nmse(seq, want):.3e}, "
          f"packed vs f64 {oracle.nmse(got, exact):.3e}, oracle vs f64 {oracle.nmse(want, exact):.3e}", flush=True)
    assert oracle.nmse(got, want) <= 1e-5
    again, _ = run_fa(pkg, gpu, q, kb, vb, mask, 0.125, pkg.FA_F16_PK)
    assert np.array_equal(again.view(np.uint32), got.view(np.uint32))          # the same bits on every run


def test_flash_attn_few_queries_take_the_f32_mask(pkg, oracle, gpu):
    # the few-query kernel reads the f32 tensor a graph would cast to f16 and rounds each value as the cast does: the same bits
    # as with the f16 copy, also for values that are not representable in f16; with more than 8 queries it says no
    lib = pkg.kernels()
    for mode, H, N, KV in [(md, *shape) for md in (pkg.FA_F16_SEQ, pkg.FA_F16_PK) for shape in ((4, 5, 300), (2, 1, 193), (3, 8, 64))]:
        q, kb, vb = _attention_inputs(oracle, H, N, KV, False, None)
        m = (RNG.normal(size=(64, KV)) * 0.37).astype(np.float32)
        m[:, KV // 2:][RNG.random((64, KV - KV // 2)) < 0.4] = -np.inf
        m[:, 0] = 0.0
        want, name = run_fa(pkg, gpu, q, kb, vb, oracle.f32_to_f16_bits(m), 0.125, mode)
        assert name == ("flash_attn.seq_row" if mode == pkg.FA_F16_SEQ else "flash_attn.seq_row_pk")
        d_q, d_k, d_v, d_m = gpu.up(q), gpu.up(kb), gpu.up(vb), gpu.up(m)
        d_o = torch.zeros((N, H, 64), dtype=torch.float32, device=gpu.dev)
        pkg.check(lib.mi355x_flash_attn_ext(pkg.tensor(d_q, pkg.F32), pkg.tensor(d_k, pkg.F16), pkg.tensor(d_v, pkg.F16), pkg.tensor(d_m, pkg.F32),
                                            pkg.tensor(d_o, pkg.F32), 0.125, mode, None, 0, gpu.stream))
        assert np.array_equal(gpu.down(d_o).view(np.uint32), want.view(np.uint32))
        # ... and leaves the f16 copy behind for later readers (rows of the queries; the rest is not touched)
        d_c = torch.full((64, KV), 7, dtype=torch.int16, device=gpu.dev)
        d_o.zero_()
        pkg.check(lib.mi355x_flash_attn_ext_cast_mask(pkg.tensor(d_q, pkg.F32), pkg.tensor(d_k, pkg.F16), pkg.tensor(d_v, pkg.F16), pkg.tensor(d_m, pkg.F32),
                                                      pkg.tensor(d_c, pkg.F16), pkg.tensor(d_o, pkg.F32), 0.125, mode, None, 0, gpu.stream))
        assert np.array_equal(gpu.down(d_o).view(np.uint32), want.view(np.uint32))
        copy = gpu.down(d_c).view(np.uint16)
        assert np.array_equal(copy[:N], oracle.f32_to_f16_bits(m)[:N]) and np.all(copy[N:] == 7)
    q, kb, vb = _attention_inputs(oracle, 2, 9, 64, False, None)
    d_m = gpu.up(np.zeros((64, 64), dtype=np.float32))
    d_o = torch.zeros((9, 2, 64), dtype=torch.float32, device=gpu.dev)
    assert lib.mi355x_flash_attn_ext(pkg.tensor(gpu.up(q), pkg.F32), pkg.tensor(gpu.up(kb), pkg.F16), pkg.tensor(gpu.up(vb), pkg.F16), pkg.tensor(d_m, pkg.F32),
                                     pkg.tensor(d_o, pkg.F32), 0.125, pkg.FA_F16_SEQ, None, 0, gpu.stream) == -1


def test_flash_attn_emits_the_next_products_activation_image(pkg, oracle, gpu):
    # MI355X_FA_EMIT_F16: besides dst, the rows [N][H * 64] rounded to Q8_0 and stored as f16(q * d)
    H, N, KV = 4, 100, 130
    q, kb, vb = _attention_inputs(oracle, H, N, KV)
    d_q, d_k, d_v = gpu.up(q), gpu.up(kb), gpu.up(vb)
    d_o = torch.empty((N, H, 64), dtype=torch.float32, device=gpu.dev)
    d_h = torch.zeros((N, H * 64), dtype=torch.float16, device=gpu.dev)
    tq, tk, tv, to = pkg.tensor(d_q, pkg.F32), pkg.tensor(d_k, pkg.F16), pkg.tensor(d_v, pkg.F16), pkg.tensor(d_o, pkg.F32)
    lib = pkg.kernels()
    pkg.check(lib.mi355x_flash_attn_ext(tq, tk, tv, None, to, 0.125, pkg.FA_F16_SEQ | pkg.FA_EMIT_F16, d_h.data_ptr(), d_h.numel() * 2, gpu.stream))
    y = gpu.down(d_o).reshape(N, H * 64)
    assert oracle.nmse(y, oracle.flash_attn_ext(q, kb, vb, None, 0.125).reshape(N, H * 64)) <= 1e-6
    image = oracle.dequantize(oracle.Q8_0, oracle.quantize(oracle.Q8_0, y, act=True), H * 64).reshape(N, H * 64)
    assert np.array_equal(gpu.down(d_h, np.uint16), oracle.f32_to_f16_bits(image))
    # not for the few-query kernel, and not without room for the image
    d_q5 = gpu.up(q[:, :5])
    d_o5 = torch.empty((5, H, 64), dtype=torch.float32, device=gpu.dev)
    assert lib.mi355x_flash_attn_ext(pkg.tensor(d_q5, pkg.F32), tk, tv, None, pkg.tensor(d_o5, pkg.F32), 0.125, pkg.FA_EMIT_F16, d_h.data_ptr(), d_h.numel() * 2, gpu.stream) == -1
    assert lib.mi355x_flash_attn_ext(tq, tk, tv, None, to, 0.125, pkg.FA_EMIT_F16, d_h.data_ptr(), 64, gpu.stream) == -3
    # a dst without memory: the same image and nothing else; without the image, or in f32 mode, that is an error
    d_h2 = torch.zeros_like(d_h)
    t_null = pkg.tensor(d_o, pkg.F32); t_null.data = None
    d_o.fill_(7.0)
    pkg.check(lib.mi355x_flash_attn_ext(tq, tk, tv, None, t_null, 0.125, pkg.FA_F16_SEQ | pkg.FA_EMIT_F16, d_h2.data_ptr(), d_h2.numel() * 2, gpu.stream))
    assert np.array_equal(gpu.down(d_h2, np.uint16), gpu.down(d_h, np.uint16)) and np.all(gpu.down(d_o) == 7.0)
    assert lib.mi355x_flash_attn_ext(tq, tk, tv, None, t_null, 0.125, pkg.FA_F16_SEQ, None, 0, gpu.stream) == -2
    assert lib.mi355x_flash_attn_ext(tq, tk, tv, None, t_null, 0.125, pkg.FA_F32 | pkg.FA_EMIT_F16, d_h2.data_ptr(), d_h2.numel() * 2, gpu.stream) == -2


def test_flash_attn_few_queries_emit_q8_0(pkg, oracle, gpu):
    # MI355X_FA_EMIT_Q8_0: a decode step's attention leaves its rows [N][H * 64] quantized for the projection that follows
    H, N, KV = 6, 5, 200
    q, kb, vb = _attention_inputs(oracle, H, N, KV)
    d_q, d_k, d_v = gpu.up(q), gpu.up(kb), gpu.up(vb)
    d_o = torch.empty((N, H, 64), dtype=torch.float32, device=gpu.dev)
    k = H * 64
    d_w = torch.zeros(N * k + N * (k // 32) * 8, dtype=torch.uint8, device=gpu.dev)
    tq, tk, tv, to = pkg.tensor(d_q, pkg.F32), pkg.tensor(d_k, pkg.F16), pkg.tensor(d_v, pkg.F16), pkg.tensor(d_o, pkg.F32)
    lib = pkg.kernels()
    for mode, bound in ((pkg.FA_F16_SEQ, 1e-6), (pkg.FA_F16_PK, 1e-5)):
        d_w.zero_()
        pkg.check(lib.mi355x_flash_attn_ext(tq, tk, tv, None, to, 0.125, mode | pkg.FA_EMIT_Q8_0, d_w.data_ptr(), d_w.numel(), gpu.stream))
        y, image = gpu.down(d_o).reshape(N, k), gpu.down(d_w)
        assert oracle.nmse(y, oracle.flash_attn_ext(q, kb, vb, None, 0.125).reshape(N, k)) <= bound
        want = oracle.quantize(oracle.Q8_0, y, act=True).reshape(N, k // 32, 34)
        assert np.array_equal(image[: N * k].reshape(N, k // 32, 32), want[:, :, 2:])
        assert np.array_equal(image[N * k : N * k + N * (k // 32) * 4].view(np.float32).reshape(N, k // 32),
                              oracle.f16_bits_to_f32(want[:, :, :2].copy().view(np.uint16)[..., 0]))
        assert np.array_equal(image[N * k + N * (k // 32) * 4 :].view(np.int32).reshape(N, k // 32), want[:, :, 2:].view(np.int8).astype(np.int32).sum(-1))
    # the many-query kernels do not write this form
    d_q9 = gpu.up(rnd((H, 9, 64)))
    d_o9 = torch.empty((9, H, 64), dtype=torch.float32, device=gpu.dev)
    assert lib.mi355x_flash_attn_ext(pkg.tensor(d_q9, pkg.F32), tk, tv, None, pkg.tensor(d_o9, pkg.F32), 0.125, pkg.FA_EMIT_Q8_0, d_w.data_ptr(), d_w.numel(), gpu.stream) == -1


def _attention_float64(oracle, q, kb, vb, mask, scale):
    qf = oracle.f16_bits_to_f32(oracle.f32_to_f16_bits(q)).astype(np.float64)
    s = np.einsum("hnd,hkd->hnk", qf, oracle.f16_bits_to_f32(kb).astype(np.float64)) * scale
    if mask is not None:
        s = s + oracle.f16_bits_to_f32(mask)[None, : q.shape[1]].astype(np.float64)
    p = np.exp(s - s.max(-1, keepdims=True)); p /= p.sum(-1, keepdims=True)
    return np.einsum("hnk,hkd->nhd", p, oracle.f16_bits_to_f32(vb).astype(np.float64))


@pytest.mark.parametrize("case", [
    dict(H=2, N=5, KV=300, flat=True, pad_from=280), dict(H=2, N=30, KV=300, flat=True, pad_from=280), dict(H=3, N=200, KV=1536, flat=True, pad_from=1500),
    dict(H=2, N=70, KV=100), dict(H=2, N=9, KV=63), dict(H=2, N=33, KV=37, mask="beam"), dict(H=2, N=100, KV=100, mask="causal"),
    dict(H=2, N=130, KV=448, mask="causal"), dict(H=1, N=64, KV=20)])
def test_flash_attn_f32_mode_matches_float64(pkg, oracle, gpu, case):
    # MI355X_FA_F32: f32 accumulators.  More than 8 queries: both products on the matrix cores, probabilities rounded to f16
    # (relative 2^-11 each, averaged over the keys); otherwise plain f32 arithmetic.
    H, N, KV = case["H"], case["N"], case["KV"]
    q, kb, vb = _attention_inputs(oracle, H, N, KV, case.get("flat", False), case.get("pad_from"))
    mask = None
    if "mask" in case:
        m = np.full((-(-N // 64) * 64, KV), -np.inf, dtype=np.float32)
        for r in range(N):
            if case["mask"] == "causal":
                m[r, : KV - N + r + 1] = 0.0
            else:
                m[r, : (KV + 1) // 2] = 0.0
                m[r, [c for c in range(KV) if c % N == r]] = 0.0
        mask = oracle.f32_to_f16_bits(m)
    got, name = run_fa(pkg, gpu, q, kb, vb, mask, 0.125, pkg.FA_F32)
    assert name == ("flash_attn.mfma_f32" if N > 8 else "flash_attn.vec_f32")
    assert np.isfinite(got).all()
    exact = _attention_float64(oracle, q, kb, vb, mask, 0.125)
    assert oracle.nmse(got, exact) <= (1e-7 if N > 8 else 1e-9)
    # north-star per-op bound against the CPU backend's own arithmetic (f16 accumulator rounded after every key)
    assert oracle.nmse(got, oracle.flash_attn_ext(q, kb, vb, None if mask is None else mask[:N], 0.125)) <= 5e-4


def test_flash_attn_f32_mode_emits_the_activation_image(pkg, oracle, gpu):
    H, N, KV = 4, 100, 130
    q, kb, vb = _attention_inputs(oracle, H, N, KV)
    d_q, d_k, d_v = gpu.up(q), gpu.up(kb), gpu.up(vb)
    d_o = torch.empty((N, H, 64), dtype=torch.float32, device=gpu.dev)
    d_h = torch.zeros((N, H * 64), dtype=torch.float16, device=gpu.dev)
    tq, tk, tv, to = pkg.tensor(d_q, pkg.F32), pkg.tensor(d_k, pkg.F16), pkg.tensor(d_v, pkg.F16), pkg.tensor(d_o, pkg.F32)
    pkg.check(pkg.kernels().mi355x_flash_attn_ext(tq, tk, tv, None, to, 0.125, pkg.FA_F32 | pkg.FA_EMIT_F16, d_h.data_ptr(), d_h.numel() * 2, gpu.stream))
    y = gpu.down(d_o).reshape(N, H * 64)
    assert oracle.nmse(y, _attention_float64(oracle, q, kb, vb, None, 0.125).reshape(N, H * 64)) <= 1e-7
    image = oracle.dequantize(oracle.Q8_0, oracle.quantize(oracle.Q8_0, y, act=True), H * 64).reshape(N, H * 64)
    assert np.array_equal(gpu.down(d_h, np.uint16), oracle.f32_to_f16_bits(image))


def test_flash_attn_strided_views_like_whisper(pkg, oracle, gpu):
    # Q is the permuted view of a [d, N] projection; K / V are slices of a 1-d cache with row pitch d (src/whisper.cpp:2149-2172):
    # many queries and a decode step's few, both forms of the step, and grouped heads (two query heads to a K / V head)
    for N, KV, mode, bound, HKV in ((20, 96, "FA_F16_SEQ", 1e-6, 4), (20, 96, "FA_F16_PK", 1e-5, 4), (5, 500, "FA_F16_SEQ", 1e-6, 4), (5, 500, "FA_F16_PK", 1e-5, 4),
                                    (3, 333, "FA_F16_PK", 1e-5, 2), (3, 333, "FA_F16_SEQ", 1e-6, 2)):
        H, D = 4, 64
        d, dkv = H * D, HKV * D
        qcur, kc, vc = rnd((N, d)), rnd((KV, dkv)), rnd((KV, dkv))
        d_q, d_k, d_v = gpu.up(qcur), gpu.up(oracle.f32_to_f16_bits(kc)), gpu.up(oracle.f32_to_f16_bits(vc))
        d_o = torch.empty((N, H, D), dtype=torch.float32, device=gpu.dev)
        tq = pkg.tensor(d_q, pkg.F32, ne=[D, N, H], nb=[4, d * 4, D * 4, d * 4 * N])
        tk = pkg.tensor(d_k, pkg.F16, ne=[D, KV, HKV], nb=[2, dkv * 2, D * 2, dkv * 2 * KV])
        tv = pkg.tensor(d_v, pkg.F16, ne=[D, KV, HKV], nb=[2, dkv * 2, D * 2, dkv * 2 * KV])
        pkg.check(pkg.kernels().mi355x_flash_attn_ext(tq, tk, tv, None, pkg.tensor(d_o, pkg.F32), 0.125, getattr(pkg, mode), None, 0, gpu.stream))
        q = qcur.reshape(N, H, D).transpose(1, 0, 2)
        kb = np.repeat(oracle.f32_to_f16_bits(kc).reshape(KV, HKV, D).transpose(1, 0, 2), H // HKV, axis=0)
        vb = np.repeat(oracle.f32_to_f16_bits(vc).reshape(KV, HKV, D).transpose(1, 0, 2), H // HKV, axis=0)
        assert oracle.nmse(gpu.down(d_o), oracle.flash_attn_ext(q, np.ascontiguousarray(kb), np.ascontiguousarray(vb), None, 0.125)) <= bound, (N, KV, mode, HKV)


# ------------------------------------------------------------------------------------------------------------------

def test_norm_and_affine(pkg, oracle, gpu):
    lib = pkg.kernels()
    for shape in [(1500, 1280), (7, 100), (3, 5000), (5, 512)]:
        x = rnd(shape, 2.0, 0.3)
        d_x = gpu.up(x)
        d_y = torch.empty_like(d_x)
        pkg.check(lib.mi355x_norm(pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32), 1e-5, None, None, gpu.stream))
        want = oracle.norm(x, 1e-5)
        assert oracle.nmse(gpu.down(d_y), want) <= 1e-10
        w, b = rnd((shape[1],), 0.02, 1.0), rnd((shape[1],), 0.02)
        d_w, d_b = gpu.up(w), gpu.up(b)
        pkg.check(lib.mi355x_norm(pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32), 1e-5, d_w.data_ptr(), d_b.data_ptr(), gpu.stream))
        assert oracle.nmse(gpu.down(d_y), want * w + b) <= 1e-10
        # the variant that also leaves the GEMM's activation image: the Q8_0 rounding of what it just wrote, as f16(q * d)
        d_h = torch.zeros(shape, dtype=torch.float16, device=gpu.dev)
        rc = lib.mi355x_norm_emit_f16(pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32), 1e-5, d_w.data_ptr(), d_b.data_ptr(), d_h.data_ptr(), gpu.stream)
        if shape[1] % 32 == 0 and shape[1] <= 2048:
            pkg.check(rc)
            y = gpu.down(d_y)
            assert oracle.nmse(y, want * w + b) <= 1e-10
            image = oracle.dequantize(oracle.Q8_0, oracle.quantize(oracle.Q8_0, y, act=True), shape[1]).reshape(shape)
            assert np.array_equal(gpu.down(d_h, np.uint16), oracle.f32_to_f16_bits(image))
            # without a destination (data pointer NULL): the same image and no other store
            t_null = pkg.tensor(d_y, pkg.F32); t_null.data = None
            d_h2 = torch.zeros(shape, dtype=torch.float16, device=gpu.dev)
            d_y.fill_(7.0)
            pkg.check(lib.mi355x_norm_emit_f16(pkg.tensor(d_x, pkg.F32), t_null, 1e-5, d_w.data_ptr(), d_b.data_ptr(), d_h2.data_ptr(), gpu.stream))
            assert np.array_equal(gpu.down(d_h2, np.uint16), gpu.down(d_h, np.uint16)) and np.all(gpu.down(d_y) == 7.0)
        else:
            assert rc == -1                      # unsupported shapes say so; the caller falls back to the plain kernel
        # and the variant for the few-column product: Q8_0 itself, quants | scales | block sums
        n, k = shape
        d_q = torch.zeros(n * k + n * (k // 32 + 1) * 8, dtype=torch.uint8, device=gpu.dev)
        rc = lib.mi355x_norm_emit_q8_0(pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32), 1e-5, d_w.data_ptr(), d_b.data_ptr(), d_q.data_ptr(), gpu.stream)
        if k % 32 == 0 and k <= 2048:
            pkg.check(rc)
            y, image = gpu.down(d_y), gpu.down(d_q)
            q = oracle.quantize(oracle.Q8_0, y, act=True).reshape(n, k // 32, 34)
            assert np.array_equal(image[: n * k].reshape(n, k // 32, 32), q[:, :, 2:])
            assert np.array_equal(image[n * k : n * k + n * (k // 32) * 4].view(np.float32).reshape(n, k // 32),
                                  oracle.f16_bits_to_f32(q[:, :, :2].copy().view(np.uint16)[..., 0]))
            sums = image[n * k + n * (k // 32) * 4 : n * k + n * (k // 32) * 8].view(np.int32).reshape(n, k // 32)
            assert np.array_equal(sums, q[:, :, 2:].view(np.int8).astype(np.int32).sum(-1))
        else:
            assert rc == -1


def test_gelu_scale_binary(pkg, oracle, gpu):
    lib = pkg.kernels()
    x = rnd((1500, 640), 3.0)
    d_x = gpu.up(x)
    d_y = torch.empty_like(d_x)
    pkg.check(lib.mi355x_gelu(pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32), gpu.stream))
    got, want = gpu.down(d_y), oracle.gelu(x)
    assert oracle.nmse(got, want) <= 1e-7 and np.mean(got != want) < 0.02       # same f16-table semantics; exp() ulps flip a few f16 roundings
    pkg.check(lib.mi355x_scale(pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32), 0.35355339, gpu.stream))
    assert np.array_equal(gpu.down(d_y), oracle.scale(x, 0.35355339))
    a = rnd((6, 5, 7))
    for op in (0, 1):
        for bshape in [(6, 5, 7), (7,), (1, 5, 1), (6, 1, 7), (3, 1, 7)]:
            b = rnd(bshape)
            d_a, d_b = gpu.up(a), gpu.up(b)
            d_o = torch.empty_like(d_a)
            pkg.check(lib.mi355x_binary(op, pkg.tensor(d_a, pkg.F32), pkg.tensor(d_b, pkg.F32), pkg.tensor(d_o, pkg.F32), gpu.stream))
            assert np.array_equal(gpu.down(d_o), oracle.binary(op, a, b))
    # in place, big, row vector (bias add of whisper)
    big, bias = rnd((1500, 1280)), rnd((1280,))
    d_a, d_b = gpu.up(big), gpu.up(bias)
    pkg.check(lib.mi355x_binary(0, pkg.tensor(d_a, pkg.F32), pkg.tensor(d_b, pkg.F32), pkg.tensor(d_a, pkg.F32), gpu.stream))
    assert np.array_equal(gpu.down(d_a), big + bias)


def test_cpy_get_rows_im2col_softmax_concat(pkg, oracle, gpu):
    lib = pkg.kernels()
    # f32 -> f16 dense and transposed
    x = rnd((1500, 320))
    d_x = gpu.up(x)
    d_h = torch.empty(x.shape, dtype=torch.float16, device=gpu.dev)
    pkg.check(lib.mi355x_cpy(pkg.tensor(d_x, pkg.F32), pkg.tensor(d_h, pkg.F16), gpu.stream))
    assert np.array_equal(gpu.down(d_h).view(np.uint16), oracle.f32_to_f16_bits(x))
    d_t = torch.empty((320, 1500), dtype=torch.float32, device=gpu.dev)
    pkg.check(lib.mi355x_cpy(pkg.tensor(d_x.t(), pkg.F32), pkg.tensor(d_t, pkg.F32), gpu.stream))     # CONT of a transposed view
    assert np.array_equal(gpu.down(d_t), x.T)
    # get_rows
    w = rnd((300, 128), 0.02)
    ids = np.array([5, 299, 0, 5, 17], dtype=np.int32)
    for t in (pkg.Q5_0, pkg.Q8_0):
        blocks = oracle.quantize(t, w)
        d_w, d_i = gpu.up(blocks), gpu.up(ids)
        d_o = torch.empty((5, 128), dtype=torch.float32, device=gpu.dev)
        pkg.check(lib.mi355x_get_rows(pkg.tensor(d_w, t, ne=[128, 300]), pkg.tensor(d_i, pkg.I32), pkg.tensor(d_o, pkg.F32), gpu.stream))
        assert np.array_equal(gpu.down(d_o), oracle.get_rows(t, blocks, ids, 128))
        # the token + positional embedding of a decoder input as one launch: the same gathers and the same f32 sum
        pos_table, pos = rnd((40, 128)), np.array([7, 8, 39, 0, 7], dtype=np.int32)
        d_p, d_pi = gpu.up(pos_table), gpu.up(pos)
        d_o.fill_(3.0)
        pkg.check(lib.mi355x_get_rows_add(pkg.tensor(d_w, t, ne=[128, 300]), pkg.tensor(d_i, pkg.I32), pkg.tensor(d_p, pkg.F32), pkg.tensor(d_pi, pkg.I32),
                                          pkg.tensor(d_o, pkg.F32), gpu.stream))
        assert np.array_equal(gpu.down(d_o), oracle.binary(0, oracle.get_rows(t, blocks, ids, 128), pos_table[pos]))
        assert lib.mi355x_get_rows_add(pkg.tensor(d_w, t, ne=[128, 300]), pkg.tensor(d_i, pkg.I32), pkg.tensor(d_p, pkg.F32), pkg.tensor(d_pi[:4], pkg.I32),
                                       pkg.tensor(d_o, pkg.F32), gpu.stream) == -1
        # an index outside the matrix (the reference aborts on it, ops.cpp:4174) reads nothing and gives a NaN row; the rows
        # beside it are what they were
        bad = np.array([5, 300, 0, -1, 17], dtype=np.int32)
        d_b = gpu.up(bad)
        pkg.check(lib.mi355x_get_rows(pkg.tensor(d_w, t, ne=[128, 300]), pkg.tensor(d_b, pkg.I32), pkg.tensor(d_o, pkg.F32), gpu.stream))
        got = gpu.down(d_o)
        assert np.isnan(got[[1, 3]]).all() and np.array_equal(got[[0, 2, 4]], oracle.get_rows(t, blocks, ids, 128)[[0, 2, 4]])
        pkg.check(lib.mi355x_get_rows_add(pkg.tensor(d_w, t, ne=[128, 300]), pkg.tensor(d_i, pkg.I32), pkg.tensor(d_p, pkg.F32), pkg.tensor(gpu.up(np.array([7, 8, 40, 0, -3], dtype=np.int32)), pkg.I32),
                                          pkg.tensor(d_o, pkg.F32), gpu.stream))
        got = gpu.down(d_o)
        assert np.isnan(got[[2, 4]]).all() and np.array_equal(got[[0, 1, 3]], oracle.binary(0, oracle.get_rows(t, blocks, ids, 128), pos_table[pos])[[0, 1, 3]])
    # im2col, the two strides of the conv stem, odd sizes
    src = rnd((33, 77))
    for s0 in (1, 2):
        want = oracle.im2col_1d(src, 3, s0, 1, 1)
        d_s = gpu.up(src)
        d_o = torch.empty(want.shape, dtype=torch.float16, device=gpu.dev)
        pkg.check(lib.mi355x_im2col_1d(pkg.tensor(d_s, pkg.F32), pkg.tensor(d_o, pkg.F16), 3, s0, 1, 1, gpu.stream))
        assert np.array_equal(gpu.down(d_o).view(np.uint16), want)
    # soft_max with an f32 mask shared by all heads
    kq = rnd((4, 5, 37), 3.0)
    mask = np.zeros((64, 37), dtype=np.float32); mask[:, 30:] = -np.inf
    d_k, d_m = gpu.up(kq), gpu.up(mask)
    d_o = torch.empty_like(d_k)
    pkg.check(lib.mi355x_soft_max(pkg.tensor(d_k, pkg.F32), pkg.tensor(d_m, pkg.F32), pkg.tensor(d_o, pkg.F32), 0.125, gpu.stream))
    assert oracle.nmse(gpu.down(d_o), oracle.soft_max(kq, mask[:5], 0.125)) <= 1e-10
    # concat along ggml dim 2
    a, b = rnd((2, 5, 30)), rnd((3, 5, 30))
    d_a, d_b = gpu.up(a), gpu.up(b)
    d_o = torch.empty((5, 5, 30), dtype=torch.float32, device=gpu.dev)
    pkg.check(lib.mi355x_concat(pkg.tensor(d_a, pkg.F32), pkg.tensor(d_b, pkg.F32), pkg.tensor(d_o, pkg.F32), 2, gpu.stream))
    assert np.array_equal(gpu.down(d_o), np.concatenate([a, b], axis=0))


# ------------------------------------------------------------------------------------------------------------------
# the committed vectors of the reference's CPU backend (tests/golden), on the GPU box where the reference does not exist
# ------------------------------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def vec():
    from pathlib import Path
    return np.load(Path(__file__).resolve().parent / "golden" / "cpu_backend_vectors.npz", allow_pickle=False)


@pytest.mark.parametrize("name", ["q5_0", "q8_0"])
def test_golden_dequantize_and_mul_mat(pkg, oracle, gpu, vec, name):
    t = getattr(pkg, name.upper())
    blocks = vec[f"quant_{name}_blocks"]
    d_b = gpu.up(blocks)
    d_y = torch.empty(blocks.shape[0] * 128, dtype=torch.float32, device=gpu.dev)
    pkg.check(pkg.kernels().mi355x_dequantize_row(t, d_b.data_ptr(), d_y.data_ptr(), d_y.numel(), gpu.stream))
    assert np.array_equal(gpu.down(d_y).view(np.uint32), vec[f"dequant_{name}"].reshape(-1).view(np.uint32))       # bit-exact
    for n in (1, 5, 40):
        got, kernel = run_mul_mat(pkg, gpu, t, vec[f"mul_mat_{name}_w"], vec[f"mul_mat_{name}_x_n{n}"], 128, 48)
        # north-star bound 5e-4; the GEMV forms the reference's integers (1e-10), the GEMM rounds d*q to f16 (1e-6)
        assert oracle.nmse(got, vec[f"mul_mat_{name}_y_n{n}"]) <= (1e-10 if "gemv" in kernel else 1e-6), kernel


def test_golden_activation_quantizer(pkg, gpu, vec):
    x = vec["act_q8_0_input"]
    d_x = gpu.up(x)
    d_q = torch.empty(x.size // 32 * 34, dtype=torch.uint8, device=gpu.dev)
    pkg.check(pkg.kernels().mi355x_quantize_row_q8_0(d_x.data_ptr(), d_q.data_ptr(), x.size, gpu.stream))
    assert np.array_equal(gpu.down(d_q).reshape(x.shape[0], -1), vec["act_q8_0_blocks"])


@pytest.mark.parametrize("name", ["enc", "dec"])
def test_golden_flash_attn(pkg, oracle, gpu, vec, name):
    mask = vec[f"fa_{name}_mask"] if f"fa_{name}_mask" in vec else None
    got, _ = run_fa(pkg, gpu, vec[f"fa_{name}_q"], vec[f"fa_{name}_k"], vec[f"fa_{name}_v"], mask, float(vec[f"fa_{name}_scale"]), pkg.FA_F16_SEQ)
    assert oracle.nmse(got, vec[f"fa_{name}_y"]) <= 1e-6           # north-star bound 5e-4


def test_golden_norm_gelu_soft_max(pkg, oracle, gpu, vec):
    lib = pkg.kernels()
    for op, x, want, tol in (("norm", vec["norm_x"], vec["norm_y"], 1e-12), ("gelu", vec["gelu_x"], vec["gelu_y"], 0.0),
                             ("soft_max", vec["soft_max_x"], vec["soft_max_y"], 1e-12)):
        d_x = gpu.up(x)
        d_y = torch.empty_like(d_x)
        tx, ty = pkg.tensor(d_x, pkg.F32), pkg.tensor(d_y, pkg.F32)
        if op == "norm":
            pkg.check(lib.mi355x_norm(tx, ty, 1e-5, None, None, gpu.stream))
        elif op == "gelu":
            pkg.check(lib.mi355x_gelu(tx, ty, gpu.stream))
        else:
            pkg.check(lib.mi355x_soft_max(tx, None, ty, float(vec["soft_max_scale"]), gpu.stream))
        got = gpu.down(d_y)
        if tol == 0.0:
            assert np.array_equal(got, want), op                 # the f16 table makes GELU reproducible bit for bit
        else:
            assert oracle.nmse(got, want) <= tol, op


def test_smoke_entry_point():
    import __graft_entry__ as entry
    entry.smoke()


# ------------------------------------------------------------------------------------------------------------------
# log-mel front end
# ------------------------------------------------------------------------------------------------------------------

def run_log_mel(pkg, gpu, samples, filters):
    lib = pkg.kernels()
    d_s, d_f = gpu.up(samples), gpu.up(filters)
    n_mel, n_len = filters.shape[0], lib.mi355x_log_mel_n_len(samples.size)
    d_mel = torch.full((n_mel, n_len), 99.0, dtype=torch.float32, device=gpu.dev)
    ws = torch.empty(lib.mi355x_log_mel_workspace_size(n_mel), dtype=torch.uint8, device=gpu.dev)
    pkg.check(lib.mi355x_log_mel_spectrogram(d_s.data_ptr(), samples.size, d_f.data_ptr(), n_mel, d_mel.data_ptr(), ws.data_ptr(), ws.numel(), gpu.stream), "log_mel")
    return gpu.down(d_mel)


def mel_test_signal(n, seed):
    r = np.random.default_rng(seed)
    t = np.arange(n) / 16000.0
    s = 0.3 * np.sin(2 * np.pi * 440.0 * t) + 0.1 * np.sin(2 * np.pi * (300.0 + 2000.0 * t) * t) + 0.01 * r.normal(size=n)
    s[: n // 5] *= 1e-2
    return s.astype(np.float32)


# Tolerance: the kernel evaluates the transform in f64, the reference in f32 (halving scheme); on the output's scale
# ((log10 power + 4) / 4, values in about [-1, 1.5]) the two agree to 1e-4 absolute, NMSE <= 1e-8.
@pytest.mark.parametrize("n,n_mel", [(201, 80), (16000 + 123, 80), (8001, 128), (160 * 16 * 7 - 200, 128), (480000, 128), (480000, 80)])
def test_log_mel_against_the_oracle(pkg, oracle, gpu, n, n_mel):
    s, f = mel_test_signal(n, n), oracle.mel_filter_bank(n_mel)
    got, want = run_log_mel(pkg, gpu, s, f), oracle.log_mel_spectrogram(s, f)
    assert got.shape == want.shape == (n_mel, (n + 480000) // 160)
    assert np.max(np.abs(got - want)) <= 1e-4
    assert oracle.nmse(got, want) <= 1e-8


def test_log_mel_golden_vectors(pkg, gpu):
    from test_golden import mel_cases
    for _, samples, filters, want in mel_cases():
        got = run_log_mel(pkg, gpu, samples, filters)
        assert got.shape == want.shape
        assert np.max(np.abs(got - want)) <= 1e-4


def test_log_mel_properties_and_arguments(pkg, oracle, gpu):
    lib = pkg.kernels()
    f = oracle.mel_filter_bank(80)
    s = mel_test_signal(48000, 3)
    a = run_log_mel(pkg, gpu, s, f)
    # scaling the signal shifts log10 power by a constant before the clamp: (x + 4) / 4 moves by log10(g^2) / 4 everywhere
    b = run_log_mel(pkg, gpu, (s * 4.0).astype(np.float32), f)
    assert np.max(np.abs((b - a) - np.log10(16.0) / 4.0)) <= 1e-5
    # the same call twice gives the same bits (the maximum is the only value formed by atomics, and a maximum has no order)
    assert np.array_equal(a.view(np.uint32), run_log_mel(pkg, gpu, s, f).view(np.uint32))
    # silence: every value is the clamp floor of the reference, (log10(1e-10) + 4) / 4
    z = run_log_mel(pkg, gpu, np.zeros(4000, dtype=np.float32), f)
    assert np.all(z == np.float32(-1.5))
    # arguments it does not take
    d = torch.zeros(1024, dtype=torch.float32, device=gpu.dev)
    assert lib.mi355x_log_mel_workspace_size(129) == 0 and lib.mi355x_log_mel_n_len(480000) == 6000
    assert lib.mi355x_log_mel_spectrogram(d.data_ptr(), 200, d.data_ptr(), 80, d.data_ptr(), d.data_ptr(), 4096, gpu.stream) == -2
    assert lib.mi355x_log_mel_spectrogram(d.data_ptr(), 1000, d.data_ptr(), 129, d.data_ptr(), d.data_ptr(), 4096, gpu.stream) == -1
    assert lib.mi355x_log_mel_spectrogram(d.data_ptr(), 1000, d.data_ptr(), 80, d.data_ptr(), None, 0, gpu.stream) == -3


def test_measurement_probes_run_and_reject_bad_arguments(pkg, gpu):
    # the yardstick kernels of the benchmark live in a library of their own (csrc/harness/probes.hip), not in the product's:
    # a bare read stream, the matrix instruction from registers, and the stamped read
    import ctypes as C
    from pathlib import Path
    assert not hasattr(pkg.kernels(), "mi355x_read_probe") and not hasattr(pkg.kernels(), "mi355x_probe_read")
    lib = C.CDLL(str(Path(pkg.__file__).resolve().parent / "lib" / "libmi355x_probes.so"))
    P = C.c_void_p
    lib.mi355x_probe_read.restype, lib.mi355x_probe_read.argtypes = C.c_int, [P, C.c_size_t, P, C.c_int, P]
    lib.mi355x_probe_read_stamped.restype, lib.mi355x_probe_read_stamped.argtypes = C.c_int64, [P, C.c_size_t, P, C.c_int, P, P]
    lib.mi355x_probe_mfma.restype, lib.mi355x_probe_mfma.argtypes = C.c_int, [C.c_int, C.c_int, P, P]
    out = torch.zeros(4, dtype=torch.int32, device=gpu.dev)
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device=gpu.dev)
    pkg.check(lib.mi355x_probe_read(buf.data_ptr(), buf.numel(), out.data_ptr(), 64, gpu.stream))
    pkg.check(lib.mi355x_probe_mfma(100, 256, out.data_ptr(), gpu.stream))
    torch.cuda.synchronize()
    assert int(out.abs().sum()) == 0                       # neither writes its sink
    assert lib.mi355x_probe_mfma(0, 256, out.data_ptr(), gpu.stream) == -2
    assert lib.mi355x_probe_mfma(100, 0, out.data_ptr(), gpu.stream) == -2
    assert lib.mi355x_probe_mfma(100, 256, None, gpu.stream) == -2
    assert lib.mi355x_probe_read(None, 16, out.data_ptr(), 64, gpu.stream) == -2
    # the stamped read: one (start, end) pair of device-clock ticks per 32 KB chunk, ends after starts
    stamps = torch.zeros(2 * (buf.numel() // 32768) + 64, dtype=torch.int64, device=gpu.dev)
    n = lib.mi355x_probe_read_stamped(buf.data_ptr(), buf.numel(), out.data_ptr(), 16, stamps.data_ptr(), gpu.stream)
    torch.cuda.synchronize()
    assert n == buf.numel() // 32768, n
    st = stamps.cpu()
    assert int(st[:n].min()) >= int(st[n:n + 16].min()) > 0        # every chunk finished after the first workgroup started
    assert lib.mi355x_probe_read_stamped(buf.data_ptr(), buf.numel(), out.data_ptr(), 16, None, gpu.stream) == -2
    # the load path of the GEMM operands: clock ticks of every workgroup's loop come back, on both paths and from all three places
    lib.mi355x_probe_load_path.restype, lib.mi355x_probe_load_path.argtypes = C.c_int, [P, C.c_size_t, C.c_int, C.c_int, C.c_int, P, P]
    src = torch.ones((4 << 20) + (1 << 20), dtype=torch.uint8, device=gpu.dev)
    for span in (0, 2 << 20, 4 << 20):
        for to_lds in (1, 0):
            clocks = torch.zeros(2 * 64 + 2, dtype=torch.int64, device=gpu.dev)
            pkg.check(lib.mi355x_probe_load_path(src.data_ptr(), span, to_lds, 50, 64, clocks.data_ptr(), gpu.stream))
            torch.cuda.synchronize()
            c = clocks.cpu()[:128].view(64, 2)
            assert int(c.min()) > 0 and 5 < float(c[:, 0].sum()) / float(c[:, 1].sum()) < 40      # 0.5 ... 4 GHz against the 100 MHz clock
            assert int(clocks[128:].abs().sum()) == 0
    assert lib.mi355x_probe_load_path(src.data_ptr(), 4096, 1, 50, 64, clocks.data_ptr(), gpu.stream) == -2
    assert lib.mi355x_probe_load_path(None, 0, 1, 50, 64, clocks.data_ptr(), gpu.stream) == -2
    assert lib.mi355x_probe_load_path(src.data_ptr(), 0, 1, 0, 64, clocks.data_ptr(), gpu.stream) == -2


def test_the_three_instruction_division_by_127_is_the_division(pkg, gpu):
    # the scale of every Q8_0 block the kernels round activations to is amax / 127.0f; they compute it as a product with the
    # reciprocal corrected once by the exact residual (div127 in csrc/kernels/common.h).  Every non-negative float, infinity
    # included, through both on the device: no result may differ.
    import ctypes as C
    from pathlib import Path
    lib = C.CDLL(str(Path(pkg.__file__).resolve().parent / "lib" / "libmi355x_probes.so"))
    lib.mi355x_probe_div127.restype, lib.mi355x_probe_div127.argtypes = C.c_int, [C.c_void_p, C.c_void_p]
    n = torch.ones(1, dtype=torch.int64, device=gpu.dev)
    pkg.check(lib.mi355x_probe_div127(n.data_ptr(), gpu.stream))
    torch.cuda.synchronize()
    assert int(n.item()) == 0

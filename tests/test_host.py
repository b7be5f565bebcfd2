"""CPU-only checks of the host side: the ABI surface of the two libraries, the synthetic-model writer against the
reference's loader and quantizers, the op-case graphs on the reference's CPU backend, and the failure modes."""
from __future__ import annotations

import re
import subprocess
import sys
from pathlib import Path

import pytest

from conftest import ROOT, run_harness


def exported(lib: Path) -> set[str]:
    out = subprocess.run(["nm", "-D", "--defined-only", str(lib)], stdout=subprocess.PIPE, text=True, check=True).stdout
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


def test_kernel_library_exports_every_declared_symbol(pkg):
    header = (ROOT / "include" / "mi355x_kernels.h").read_text()
    declared = set(re.findall(r"MI355X_API\s+[\w\s\*]+?\b(mi355x_\w+)\s*\(", header))
    assert len(declared) >= 20
    if not pkg.KERNELS_LIB.exists():
        pytest.skip("kernel library not built")
    assert declared <= exported(pkg.KERNELS_LIB), declared - exported(pkg.KERNELS_LIB)
    lib = pkg.kernels()                                # loads without a GPU; every ctypes signature binds
    assert lib.mi355x_abi_version() == 1
    assert lib.mi355x_status_string(-1).decode().startswith("unsupported")


def test_attention_refuses_a_mask_cast_that_shares_memory_with_its_output(pkg):
    # mi355x_flash_attn_ext_cast_mask reads the f32 mask while workgroups that finish early already store dst, and writes the
    # f16 copy on the way: the three may not overlap (ggml's allocator frees the f32 mask after the cast it replaces,
    # ggml/src/ggml-alloc.c:612-667, and could hand its memory to the attention node's output).  The argument checks come
    # before any HIP call, so plain addresses stand in for device memory here.
    import ctypes as C
    if not pkg.KERNELS_LIB.exists():
        pytest.skip("kernel library not built")
    lib = pkg.kernels()
    n, h, kv = 5, 20, 64
    class Mem:
        def __init__(self, addr): self.addr = addr
        def data_ptr(self): return self.addr
    def tensors(mask32_at, mask16_at, dst_at):
        q = pkg.tensor(Mem(0x10000000), pkg.F32, ne=[64, n, h], nb=[4, 256, 256 * n])
        k = pkg.tensor(Mem(0x20000000), pkg.F16, ne=[64, kv, h], nb=[2, 128, 128 * kv])
        v = pkg.tensor(Mem(0x30000000), pkg.F16, ne=[64, kv, h], nb=[2, 128, 128 * kv])
        m32 = pkg.tensor(Mem(mask32_at), pkg.F32, ne=[kv, 8], nb=[4, 4 * kv])
        m16 = pkg.tensor(Mem(mask16_at), pkg.F16, ne=[kv, 8], nb=[2, 2 * kv])
        d = pkg.tensor(Mem(dst_at), pkg.F32, ne=[64, h, n], nb=[4, 256, 256 * h])
        return q, k, v, m32, m16, d
    def call(*at):
        q, k, v, m32, m16, d = tensors(*at)
        return lib.mi355x_flash_attn_ext_cast_mask(C.byref(q), C.byref(k), C.byref(v), C.byref(m32), C.byref(m16), C.byref(d), 0.125, pkg.FA_F16_SEQ, None, 0, None)
    assert call(0x40000000, 0x40000000 + 512, 0x50000000) == -2        # the copy inside the f32 rows
    assert call(0x40000000, 0x60000000, 0x40000000 + 256) == -2        # dst over the f32 mask
    assert call(0x40000000, 0x60000000, 0x60000000) == -2              # dst over the f16 copy


def test_norm_refuses_missing_memory(pkg):
    # mi355x_norm_emit_f16 takes a destination without memory (image only); the plain and the Q8_0-emitting forms store
    # through it and must say no on the host, before any launch
    import ctypes as C
    if not pkg.KERNELS_LIB.exists():
        pytest.skip("kernel library not built")
    lib = pkg.kernels()
    class Mem:
        def __init__(self, addr): self.addr = addr
        def data_ptr(self): return self.addr
    src = pkg.tensor(Mem(0x10000000), pkg.F32, ne=[1280, 5], nb=[4, 5120])
    dst = pkg.tensor(Mem(0x20000000), pkg.F32, ne=[1280, 5], nb=[4, 5120])
    no_dst = pkg.tensor(Mem(0x20000000), pkg.F32, ne=[1280, 5], nb=[4, 5120]); no_dst.data = None
    no_src = pkg.tensor(Mem(0x10000000), pkg.F32, ne=[1280, 5], nb=[4, 5120]); no_src.data = None
    assert lib.mi355x_norm(C.byref(src), C.byref(no_dst), 1e-5, None, None, None) == -2
    assert lib.mi355x_norm(C.byref(no_src), C.byref(dst), 1e-5, None, None, None) == -2
    assert lib.mi355x_norm_emit_q8_0(C.byref(src), C.byref(no_dst), 1e-5, None, None, 0x30000000, None) == -2
    assert lib.mi355x_norm_emit_f16(C.byref(no_src), C.byref(no_dst), 1e-5, None, None, 0x30000000, None) == -2


def test_plugin_exports_the_ggml_entry_points_and_does_not_link_the_checker(pkg):
    if not pkg.PLUGIN_LIB.exists():
        pytest.skip("plugin not built")
    header = (ROOT / "include" / "ggml-mi355x.h").read_text()
    declared = set(re.findall(r"GGML_BACKEND_API\s+[\w\s\*]+?\b(ggml_backend_\w+)\s*\(", header))
    assert {"ggml_backend_init", "ggml_backend_score", "ggml_backend_mi355x_reg"} <= declared
    assert declared <= exported(pkg.PLUGIN_LIB), declared - exported(pkg.PLUGIN_LIB)
    needed = subprocess.run(["readelf", "-d", str(pkg.PLUGIN_LIB)], stdout=subprocess.PIPE, text=True, check=True).stdout
    libs = set(re.findall(r"NEEDED.*\[(.+?)\]", needed))
    assert "libmi355x_kernels.so" in libs
    # the product never links the CPU backend or the restatement: ggml-base symbols are resolved by the host process
    assert not any("ggml-cpu" in l or "oracle" in l or "whisper" in l for l in libs), libs


def test_yardstick_kernels_live_in_a_library_of_their_own(pkg):
    # the benchmark's probes are not operators: neither product library exports or needs them
    probes = pkg.KERNELS_LIB.parent / "libmi355x_probes.so"
    if not pkg.KERNELS_LIB.exists() or not probes.exists():
        pytest.skip("libraries not built")
    assert {"mi355x_probe_read", "mi355x_probe_read_stamped", "mi355x_probe_mfma", "mi355x_probe_gemv_tiles_stamped", "mi355x_probe_div127", "mi355x_probe_load_path"} <= exported(probes)
    assert not any("probe" in name for name in exported(pkg.KERNELS_LIB)), [n for n in exported(pkg.KERNELS_LIB) if "probe" in n]
    assert "probe" not in (ROOT / "include" / "mi355x_kernels.h").read_text()
    for lib in (pkg.KERNELS_LIB, pkg.PLUGIN_LIB):
        if lib.exists():
            needed = subprocess.run(["readelf", "-d", str(lib)], stdout=subprocess.PIPE, text=True, check=True).stdout
            assert "probes" not in needed


def test_missing_extension_fails_loudly(pkg, monkeypatch, tmp_path):
    monkeypatch.setattr(pkg, "_lib", None)
    monkeypatch.setattr(pkg, "KERNELS_LIB", tmp_path / "libmi355x_kernels.so")
    with pytest.raises(pkg.MissingExtension):
        pkg.kernels()


def test_writer_quantizers_and_f16_match_the_reference(harness):
    rc, rows = run_harness(harness, ["selftest"])
    assert rc == 0 and rows[-1] == {"summary": "selftest", "failed": 0}, rows


def test_synthetic_model_is_accepted_by_the_unmodified_loader(harness, tmp_path):
    model = tmp_path / "micro-q5_0.bin"
    rc, rows = run_harness(harness, ["gen", "--arch", "micro", "--ftype", "q5_0", "--out", str(model)])
    assert rc == 0 and rows[-1]["ok"]
    # whisper_init_from_file_with_params + whisper_encode + whisper_decode on the reference's CPU backend
    rc, rows = run_harness(harness, ["bench", "--model", str(model), "--what", "encoder", "--backend", "cpu", "--reps", "1", "--warmup", "0", "--threads", "4"])
    assert rc == 0 and rows[-1]["encode_ms_median"] > 0
    rc, rows = run_harness(harness, ["bench", "--model", str(model), "--what", "decoder", "--backend", "cpu", "--reps", "1", "--warmup", "1", "--steps", "6", "--threads", "4"])
    assert rc == 0 and rows[-1]["steps"] == 6
    for ftype in ("q8_0", "f16"):
        m2 = tmp_path / f"micro-{ftype}.bin"
        run_harness(harness, ["gen", "--arch", "micro", "--ftype", ftype, "--out", str(m2)])
        rc, rows = run_harness(harness, ["bench", "--model", str(m2), "--what", "encoder", "--backend", "cpu", "--reps", "1", "--warmup", "0", "--threads", "4"])
        assert rc == 0


def test_every_op_case_builds_and_runs_on_the_cpu_backend(harness):
    rc, rows = run_harness(harness, ["ops", "--cpu-only", "--quick", "--threads", "8"], timeout=600)
    assert rc == 0
    cases = [r for r in rows if "case" in r]
    assert len(cases) >= 80 and all(r["cpu_ok"] for r in cases)


def test_bench_refuses_more_than_one_gpu():
    res = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert res.returncode == 2 and "one GPU" in res.stderr

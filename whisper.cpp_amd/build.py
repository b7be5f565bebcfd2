"""Build recipes for the MI355X backend.

Four artefacts, all written under ``whisper.cpp_amd/lib`` (git-ignored, shipped to the GPU box as built):

* ``libmi355x_kernels.so`` — the HIP kernels and their C ABI (``include/mi355x_kernels.h``).  Needs only
  hipcc; builds anywhere.
* ``libggml-mi355x.so``    — the ggml backend plugin (``include/ggml-mi355x.h``).  Compiled against the ggml
  headers of a whisper.cpp tree (``--ref`` / ``$WHISPER_CPP_ROOT``, default ``/root/reference``); its
  references to the ggml-base API stay undefined and are resolved by the host process that loads it.
* ``libmi355x_probes.so``  — measurement yardsticks that ``bench.py`` loads (``csrc/harness/probes.hip``); not part of
  the product.
* ``mi355x-harness``       — test / bench driver that links the unmodified whisper.cpp host libraries
  (built by ``oracle/Makefile``) and loads the plugin with ``ggml_backend_load``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIB = PKG / "lib"
INCLUDE = ROOT / "include"
ORACLE = ROOT / "oracle"
REF_DEFAULT = Path(os.environ.get("WHISPER_CPP_ROOT", "/root/reference"))

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed-FP32 instruction selection stays off for all device code
DEVICE_FLAGS = ["--offload-arch=" + ARCH, "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON = ["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-function", "-Wno-unused-variable"]

KERNEL_SOURCES = ["misc.hip", "elementwise.hip", "rowwise.hip", "mul_mat.hip", "flash_attn.hip", "log_mel.hip"]
BACKEND_SOURCES = ["ggml-mi355x.cpp", "graph.cpp"]
HARNESS_SOURCES = ["main.cpp", "synth_model.cpp", "op_cases.cpp", "verify.cpp"]


def _run(cmd, **kw):
    cmd = [str(c) for c in cmd]
    print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, **kw)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip():
        print(out, flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"command failed ({res.returncode}): {' '.join(cmd)}")


def _obj_dir() -> Path:
    d = LIB / "obj"
    d.mkdir(parents=True, exist_ok=True)
    return d


def build_kernels() -> Path:
    """hipcc every kernel translation unit for gfx950 and link libmi355x_kernels.so."""
    objs = []
    for src in KERNEL_SOURCES:
        obj = _obj_dir() / (src + ".o")
        _run([HIPCC, *DEVICE_FLAGS, *COMMON, "-I", INCLUDE, "-c", CSRC / "kernels" / src, "-o", obj])
        objs.append(obj)
    out = LIB / "libmi355x_kernels.so"
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-o", out, *objs])
    return out


def build_probes() -> Path:
    """the measurement yardsticks of bench.py (read stream, matrix instruction, stamped instance of the logits kernel): a
    library of their own, which no product path links"""
    out = LIB / "libmi355x_probes.so"
    _run([HIPCC, *DEVICE_FLAGS, *COMMON, "-I", INCLUDE, "-shared", "-o", out, CSRC / "harness" / "probes.hip"])
    return out


def have_reference(ref: Path = REF_DEFAULT) -> bool:
    return (ref / "ggml" / "src" / "ggml-backend-impl.h").is_file()


def build_backend(ref: Path = REF_DEFAULT) -> Path:
    """Compile the ggml plugin against the host tree's ggml headers."""
    if not have_reference(ref):
        raise RuntimeError(f"no whisper.cpp tree at {ref}: the plugin is compiled against its ggml headers")
    inc = ["-I", INCLUDE, "-I", ref / "ggml" / "include", "-I", ref / "ggml" / "src"]
    defs = ["-DGGML_SHARED", "-DGGML_BACKEND_SHARED", "-DGGML_BACKEND_BUILD", "-D_GNU_SOURCE"]
    objs = []
    for src in BACKEND_SOURCES:
        obj = _obj_dir() / (src + ".o")
        _run([HIPCC, *COMMON, *defs, *inc, "-c", CSRC / "backend" / src, "-o", obj])
        objs.append(obj)
    out = LIB / "libggml-mi355x.so"
    _run([HIPCC, "-shared", "-o", out, *objs, "-L", LIB, "-lmi355x_kernels", "-Wl,-rpath,$ORIGIN"])
    return out


def build_reference(ref: Path = REF_DEFAULT) -> Path:
    """Build the unmodified whisper.cpp host libraries and ggml CPU backend into oracle/_ref."""
    if not have_reference(ref):
        raise RuntimeError(f"no whisper.cpp tree at {ref}")
    _run(["make", "-C", ORACLE, f"REF={ref}", "-j8"])
    return ORACLE / "_ref"


def build_oracle() -> Path:
    """Compile the C restatement of the reference's CPU arithmetic (checker only)."""
    out = ORACLE / "liboracle_ops.so"
    _run(["gcc", "-O2", "-std=gnu11", "-fPIC", "-shared", "-ffp-contract=off", "-o", out, ORACLE / "oracle_ops.c", "-lm"])
    return out


def build_harness(ref: Path = REF_DEFAULT) -> Path:
    """Link the test/bench driver against the host libraries in oracle/_ref."""
    if not have_reference(ref):
        raise RuntimeError(f"no whisper.cpp tree at {ref}")
    refdir = ORACLE / "_ref"
    inc = ["-I", INCLUDE, "-I", ref / "include", "-I", ref / "ggml" / "include", "-I", ref / "ggml" / "src"]
    out = LIB / "mi355x-harness"
    srcs = [CSRC / "harness" / s for s in HARNESS_SOURCES]
    _run(["g++", "-O2", "-std=c++17", "-fopenmp", "-DGGML_SHARED", "-DGGML_BACKEND_SHARED", "-DWHISPER_SHARED", *inc, *srcs, "-o", out,
          "-L", refdir, "-lwhisper", "-lggml", "-lggml-cpu", "-lggml-base", "-ldl", "-lpthread",
          "-Wl,-rpath,$ORIGIN/../../oracle/_ref"])
    return out


def build_all(ref: Path = REF_DEFAULT) -> None:
    LIB.mkdir(parents=True, exist_ok=True)
    build_kernels()
    build_probes()
    build_oracle()
    if have_reference(ref):
        build_reference(ref)
        build_backend(ref)
        build_harness(ref)
    else:
        print(f"note: {ref} absent; keeping the prebuilt plugin, host libraries and harness", flush=True)


if __name__ == "__main__":
    target = sys.argv[1] if len(sys.argv) > 1 else "all"
    {"all": build_all, "kernels": build_kernels, "backend": build_backend, "reference": build_reference,
     "oracle": build_oracle, "harness": build_harness, "probes": build_probes}[target]()

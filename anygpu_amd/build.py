"""Build recipe for the native parts: the gfx950 kernel library (hipcc), the C++ host layer's
test harness (hipcc, host-only translation units linked against the kernel library) and the
CPU oracle used by the tests (gcc, through oracle/Makefile).

Everything is built in-tree so that the shared objects travel with the source tree:
    anygpu_amd/lib/libanygpu_hip.so     kernels + C ABI (include/anygpu_hip.h)
    anygpu_amd/lib/anygpu_host_tests    reference-style C++ test harness over Tensor<dtype, device>
    oracle/liboracle.so                 CPU oracle (test infrastructure)
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
REPO_DIR = PKG_DIR.parent
CSRC_DIR = PKG_DIR / "csrc"
HOST_DIR = PKG_DIR / "host"
LIB_DIR = PKG_DIR / "lib"
OBJ_DIR = LIB_DIR / "obj"
INCLUDE_DIR = REPO_DIR / "include"
ORACLE_DIR = REPO_DIR / "oracle"

ROCM_DIR = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))
GPU_ARCH = "gfx950"
KERNEL_SOURCES = ["softmax.hip", "conv1d.hip", "gemm_f16.hip", "gemm_f32.hip", "gemm_skinny.hip", "gemm_band.hip", "gemm_band_ncontig.hip", "gemm_band_kn_f16.hip", "gemm_band_kc_wide.hip", "gemm_repack.hip", "rmsnorm.hip", "attention.hip", "attention_f32.hip", "stream_probe.hip", "capi.hip"]

# -packed-fp32-ops is switched off on purpose: packed fp32 VALU forms are not to be generated.
DEVICE_FLAGS = [
    f"--offload-arch={GPU_ARCH}", "-O3", "-std=c++20", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc and PATH)")


def _run(cmd: list[str], quiet: bool = True) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "'-packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip() and not quiet:
        print(out)


def build_kernels(verbose: bool = False) -> Path:
    """Compile every kernel translation unit for gfx950 and link libanygpu_hip.so."""
    hipcc = _hipcc()
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    objs = []
    # the main loop of the four-wave fp16 GEMM tile is generated text (an inline-assembly block with fixed registers)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f16_ring_loop.py"), str(CSRC_DIR / "gemm_f16_ring_loop.inc")], quiet=not verbose)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f16_ring_loop.py"), str(CSRC_DIR / "gemm_f16_ring_loop_kn.inc"), "kn"], quiet=not verbose)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f16_ring_loop.py"), str(CSRC_DIR / "gemm_f16_ring_loop_8x4.inc"), "8x4"], quiet=not verbose)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f16_ring_loop.py"), str(CSRC_DIR / "gemm_f16_ring_loop_4x4.inc"), "4x4"], quiet=not verbose)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f16_ring_loop.py"), str(CSRC_DIR / "gemm_f16_ring_loop_8x4kn.inc"), "8x4kn"], quiet=not verbose)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f16_ring_loop.py"), str(CSRC_DIR / "gemm_f16_ring_loop_4x4kn.inc"), "4x4kn"], quiet=not verbose)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f32_ring_loop.py"), str(CSRC_DIR / "gemm_f32_ring_loop.inc")], quiet=not verbose)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f32_ring_loop.py"), str(CSRC_DIR / "gemm_f32_ring_loop_64.inc"), "64"], quiet=not verbose)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f32_ring_loop.py"), str(CSRC_DIR / "gemm_f32_ring_loop_kn.inc"), "kn"], quiet=not verbose)
    _run([sys.executable, str(CSRC_DIR / "gen_gemm_f32_ring_loop.py"), str(CSRC_DIR / "gemm_f32_ring_loop_64kn.inc"), "64", "kn"], quiet=not verbose)

    def compile_one(src: str) -> Path:
        obj = OBJ_DIR / (Path(src).stem + ".o")
        _run([hipcc, *DEVICE_FLAGS, f"-I{INCLUDE_DIR}", f"-I{CSRC_DIR}", "-c", str(CSRC_DIR / src), "-o", str(obj)],
             quiet=not verbose)
        return obj

    with ThreadPoolExecutor(max_workers=min(len(KERNEL_SOURCES), 6)) as pool:
        objs = list(pool.map(compile_one, KERNEL_SOURCES))
    out = LIB_DIR / "libanygpu_hip.so"
    _run([hipcc, f"--offload-arch={GPU_ARCH}", "-shared", "-fPIC", "-o", str(out), *map(str, objs)], quiet=not verbose)
    return out


def build_host_harness(verbose: bool = False) -> Path | None:
    """Compile the C++ host layer's test harness, if the host layer is present."""
    main_cpp = HOST_DIR / "harness" / "main.cpp"
    if not main_cpp.exists():
        return None
    hipcc = _hipcc()
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    sources = sorted(str(p) for p in (HOST_DIR / "core").glob("*.cpp"))
    sources += sorted(str(p) for p in (HOST_DIR / "kernels").glob("*.cpp"))
    sources += sorted(str(p) for p in (HOST_DIR / "harness").glob("*.cpp"))
    includes = [f"-I{INCLUDE_DIR}", f"-I{ROCM_DIR / 'include'}"]
    includes += [f"-I{HOST_DIR / d}" for d in ("core", "ops", "fused", "kernels", "io", "transformers", "models/gemma2", "models/zamba2", "harness")]
    out = LIB_DIR / "anygpu_host_tests"
    # host-only C++ (no device code): the ROCm clang, which knows _Float16 on x86-64
    clangxx = ROCM_DIR / "lib" / "llvm" / "bin" / "clang++"
    _run([str(clangxx), "-std=c++20", "-O2", "-DAC_WITH_ASSERT", "-D__HIP_PLATFORM_AMD__", "-Wall", "-Wno-unused-function",
          *includes, *sources, "-o", str(out), f"-L{LIB_DIR}", "-lanygpu_hip", f"-L{ROCM_DIR / 'lib'}", "-lamdhip64",
          "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{ROCM_DIR / 'lib'}"], quiet=not verbose)
    return out


def build_oracle(verbose: bool = False) -> Path:
    """Build the CPU oracle (tests only)."""
    _run(["make", "-C", str(ORACLE_DIR), "-B"], quiet=not verbose)
    return ORACLE_DIR / "liboracle.so"


def build_all(verbose: bool = False) -> dict[str, str]:
    built = {"kernels": str(build_kernels(verbose))}
    harness = build_host_harness(verbose)
    if harness is not None:
        built["host_harness"] = str(harness)
    built["oracle"] = str(build_oracle(verbose))
    return built


if __name__ == "__main__":
    for name, path in build_all(verbose="-v" in sys.argv).items():
        print(f"{name}: {path}")

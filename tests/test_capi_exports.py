"""The C ABI library loads and exports exactly what include/anygpu_hip.h declares (no compute
calls here; argument validation that needs no GPU is exercised as well)."""
import ctypes
import re
import subprocess
from pathlib import Path

import pytest

REPO = Path(__file__).resolve().parent.parent
HEADER = REPO / "include" / "anygpu_hip.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(anygpu_\w+)\s*\(", text)))


def test_header_and_binding_table_agree():
    from anygpu_amd import capi
    assert declared_functions() == sorted(capi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    from anygpu_amd import capi
    lib = capi.load()
    for name in declared_functions():
        assert getattr(lib, name) is not None
    out = subprocess.run(["nm", "-D", "--defined-only", str(capi.LIB_PATH)], capture_output=True, text=True, check=True)
    exported = set(re.findall(r"\bT (anygpu_\w+)", out.stdout))
    assert exported == set(declared_functions()), "exported symbols and header declarations differ"
    assert lib.anygpu_hip_abi_version() == 1
    assert lib.anygpu_hip_target() == b"gfx950"


def test_error_strings():
    from anygpu_amd import capi
    assert capi.error_string(0) == "success"
    for code in (-1, -2, -3, -4, -5):
        assert capi.error_string(code) not in ("", "success", "unknown anygpu error code")
    assert capi.error_string(-99) == "unknown anygpu error code"


def test_argument_validation_needs_no_gpu():
    # rejected before any runtime call: shapes, strides, NULL pointers, unsupported values
    from anygpu_amd import capi
    lib = capi.load()
    fake = ctypes.c_void_p(0x1000)      # never dereferenced: every call below is rejected first
    assert lib.anygpu_gemm_f32(fake, fake, None, fake, 4, 4, 8, 4, 4, 4, 0, 0, None) == capi.ANYGPU_ERR_BAD_STRIDE
    assert lib.anygpu_gemm_f32(fake, fake, None, fake, 4, 4, 8, 8, 4, 4, 2, 0, None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert lib.anygpu_gemm_f16_f32acc(fake, fake, None, 4, 4, 8, 8, 4, 4, 0, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert lib.anygpu_gemm_f16_f32acc(fake, fake, fake, -1, 4, 8, 8, 4, 4, 0, None) == capi.ANYGPU_ERR_BAD_SHAPE
    assert lib.anygpu_gemm_f16_f32acc(fake, fake, fake, 1 << 40, 4, 8, 8, 4, 4, 0, None) == capi.ANYGPU_ERR_TOO_LARGE
    assert lib.anygpu_softmax_rows_f16(fake, fake, 4, 16, 8, 16, 0, 0, 1.0, 0.0, 0, 0, None) == capi.ANYGPU_ERR_BAD_STRIDE
    assert lib.anygpu_softmax_rows_f16(fake, None, 4, 16, 16, 16, 0, 0, 1.0, 0.0, 0, 0, None) == capi.ANYGPU_ERR_NULL_POINTER
    assert lib.anygpu_causal_conv1d_silu_f16(fake, fake, fake, fake, 2, 3, 8, 5, None) == capi.ANYGPU_ERR_UNSUPPORTED
    assert lib.anygpu_causal_conv1d_silu_f32(fake, fake, fake, fake, 2, 3, -8, 4, None) == capi.ANYGPU_ERR_BAD_SHAPE
    # the K-split workspace: rejected before the runtime is asked for the device
    assert lib.anygpu_set_workspace(None, fake, -1) == capi.ANYGPU_ERR_BAD_SHAPE
    assert lib.anygpu_set_workspace(None, None, 4096) == capi.ANYGPU_ERR_NULL_POINTER
    assert lib.anygpu_set_workspace(None, ctypes.c_void_p(0x1010), 4096) == capi.ANYGPU_ERR_UNSUPPORTED
    # empty problems succeed without touching the device
    assert lib.anygpu_gemm_f32(None, None, None, None, 0, 4, 8, 8, 4, 4, 0, 0, None) == capi.ANYGPU_OK
    assert lib.anygpu_softmax_rows_f32(None, None, 0, 16, 16, 16, 0, 0, 1.0, 0.0, 0, 0, None) == capi.ANYGPU_OK
    assert lib.anygpu_causal_conv1d_silu_f32(None, None, None, None, 0, 3, 8, 4, None) == capi.ANYGPU_OK


def test_ops_refuse_cpu_tensors():
    torch = pytest.importorskip("torch")
    from anygpu_amd import ops
    with pytest.raises(ValueError):
        ops.tensor_softmax(torch.zeros(2, 4))
    with pytest.raises(ValueError):
        ops.tensor_mm(torch.zeros(2, 4), torch.zeros(4, 2))


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from anygpu_amd import capi
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", tmp_path / "libanygpu_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        capi.load()


def test_generated_gemm_loop_is_current(tmp_path):
    # gemm_f16_ring_loop*.inc are generated texts that are committed: they have to be what the generator beside them writes
    import sys
    csrc = REPO / "anygpu_amd" / "csrc"
    for name, form in (("gemm_f32_ring_loop.inc", []), ("gemm_f32_ring_loop_64.inc", ["64"]),
                       ("gemm_f32_ring_loop_kn.inc", ["kn"]), ("gemm_f32_ring_loop_64kn.inc", ["64", "kn"])):
        out = tmp_path / name
        subprocess.run([sys.executable, str(csrc / "gen_gemm_f32_ring_loop.py"), str(out), *form], check=True)
        assert out.read_text() == (csrc / name).read_text()
    for name, form in (("gemm_f16_ring_loop.inc", []), ("gemm_f16_ring_loop_kn.inc", ["kn"]),
                       ("gemm_f16_ring_loop_8x4.inc", ["8x4"]), ("gemm_f16_ring_loop_4x4.inc", ["4x4"]),
                       ("gemm_f16_ring_loop_8x4kn.inc", ["8x4kn"]), ("gemm_f16_ring_loop_4x4kn.inc", ["4x4kn"])):
        out = tmp_path / name
        subprocess.run([sys.executable, str(csrc / "gen_gemm_f16_ring_loop.py"), str(out), *form], check=True)
        assert out.read_text() == (csrc / name).read_text()


def _gfx950_code_objects(library: Path):
    """The gfx950 code objects inside the library's .hip_fatbin section (one clang offload bundle per source file)."""
    import struct
    import tempfile
    objcopy = Path("/opt/rocm/llvm/bin/llvm-objcopy")
    if not objcopy.exists():
        pytest.skip("llvm-objcopy not found")
    with tempfile.TemporaryDirectory() as tmp:
        fat = Path(tmp) / "fat.bin"
        subprocess.run([str(objcopy), "-O", "binary", "--only-section=.hip_fatbin", str(library), str(fat)], check=True)
        data = fat.read_bytes()
    magic = b"__CLANG_OFFLOAD_BUNDLE__"
    pos = 0
    while True:
        start = data.find(magic, pos)
        if start < 0:
            return
        (entries,) = struct.unpack_from("<Q", data, start + len(magic))
        p = start + len(magic) + 8
        for _ in range(entries):
            offset, size, triple_len = struct.unpack_from("<QQQ", data, p)
            p += 24
            triple = data[p:p + triple_len].decode()
            p += triple_len
            if "gfx950" in triple:
                yield data[start + offset:start + offset + size]
        pos = start + len(magic)


def test_kernels_use_no_scratch_memory(tmp_path):
    # A kernel with a private segment (register spills, private arrays) makes the runtime allocate scratch memory for the
    # queue at its first launch, tens of megabytes behind the caller's back.  Every kernel's metadata has to say 0 bytes,
    # except the one instantiation listed (the eight-wave 256 x 256 tile with guarded rows, a K tail and partial planes,
    # which products of that shape reach only when the four-wave kernels cannot take them).
    readelf = Path("/opt/rocm/llvm/bin/llvm-readelf")
    lib = REPO / "anygpu_amd" / "lib" / "libanygpu_hip.so"
    if not readelf.exists() or not lib.exists():
        pytest.skip("llvm-readelf or the built library not found")
    allowed = re.compile(r"gemm_f16_nt_tile_kernelINS_11GemmTileCfgILi256ELi256E.*ELb1ELb1ELb1ELin1E")
    seen, offenders = 0, []
    for k, blob in enumerate(_gfx950_code_objects(lib)):
        path = tmp_path / f"co{k}.elf"
        path.write_bytes(blob)
        notes = subprocess.run([str(readelf), "--notes", str(path)], check=True, capture_output=True, text=True).stdout
        name = None
        for line in notes.splitlines():
            line = line.strip()
            if line.startswith(".name:"):
                name = line.split(":", 1)[1].strip()
            elif line.startswith(".private_segment_fixed_size:"):
                seen += 1
                if int(line.split(":", 1)[1]) != 0 and not allowed.search(name or ""):
                    offenders.append((name, line))
    assert seen > 100, "kernel metadata not found"
    assert not offenders, offenders

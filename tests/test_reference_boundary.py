"""The drop-in boundary as compiled code, checked against the reference's own headers (skipped where the reference
tree is not mounted): every shimmed function has the reference's exact type, the backend patch applies, and the two
translation units that are built inside the reference tree compile against it."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
PATCH = os.path.join(ROOT, "include", "oil_backend_gfx950.patch")
SHIM = os.path.join(ROOT, "innova_amd", "csrc", "shim")

pytestmark = pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "include", "oil")), reason="reference tree not mounted")


def cxx(args, **kw):
    r = subprocess.run(["g++", "-std=c++20", "-fsyntax-only", "-Wall", "-Werror"] + args, capture_output=True, text=True, **kw)
    assert r.returncode == 0, r.stderr[-4000:]


def test_shim_signatures_are_the_references():
    cxx([f"-I{REF}/include", f"-I{ROOT}/include", os.path.join(ROOT, "tests", "cpp", "check_reference_signatures.cpp")])


def test_a_drifted_signature_fails_to_compile(tmp_path):
    """The check has teeth: the same translation unit with one expected type changed is rejected."""
    src = open(os.path.join(ROOT, "tests", "cpp", "check_reference_signatures.cpp")).read()
    bad = src.replace("void (*)(const u8*, const u16*, const float*, float*, int, int, int)>);",
                      "void (*)(const u8*, const u16*, const float*, float*, int, int, long)>);", 1)
    assert bad != src
    f = tmp_path / "drifted.cpp"
    f.write_text(bad)
    r = subprocess.run(["g++", "-std=c++20", "-fsyntax-only", f"-I{REF}/include", f"-I{ROOT}/include", str(f)],
                       capture_output=True, text=True)
    assert r.returncode != 0 and "static assertion failed" in r.stderr


def test_backend_patch_applies_to_the_reference():
    r = subprocess.run(["patch", "--dry-run", "-p1", "-d", REF, "-i", PATCH], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "include/oil/backend.h" in r.stdout and "src/backend.cpp" in r.stdout


@pytest.fixture
def patched_tree(tmp_path):
    """backend.h / backend.cpp with the patch applied, in a temporary directory."""
    os.makedirs(tmp_path / "include" / "oil")
    os.makedirs(tmp_path / "src")
    shutil.copy(os.path.join(REF, "include", "oil", "backend.h"), tmp_path / "include" / "oil")
    shutil.copy(os.path.join(REF, "src", "backend.cpp"), tmp_path / "src")
    subprocess.run(["patch", "-s", "-p1", "-d", str(tmp_path), "-i", PATCH], check=True)
    return tmp_path


def test_reference_tree_sources_compile(patched_tree):
    inc = [f"-I{patched_tree}/include", f"-I{REF}/include", f"-I{ROOT}/include", "-I/opt/rocm/include",
           "-D__HIP_PLATFORM_AMD__", "-DOIL_USE_HIP_GFX950"]
    cxx(inc + [os.path.join(SHIM, "oil_backend_gfx950.cpp")])
    cxx(inc + [os.path.join(SHIM, "oil_engines_gfx950.cpp")])
    cxx(inc + ["-x", "c++", os.path.join(SHIM, "oil_shims.cpp")])
    # the patched dispatch itself (the reference's own file: warnings are its business)
    r = subprocess.run(["g++", "-std=c++20", "-fsyntax-only", "-w"] + inc + [str(patched_tree / "src" / "backend.cpp")],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    text = open(patched_tree / "src" / "backend.cpp").read()
    assert "case BackendType::GPU_HIP_GFX950" in text and "hw.has_hip_gfx950" in text


ENGINE_PATCH = os.path.join(ROOT, "include", "qwen35_engine_gfx950.patch")


def test_engine_patch_applies_to_the_reference():
    r = subprocess.run(["patch", "--dry-run", "-p1", "-d", REF, "-i", ENGINE_PATCH], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "include/oil/qwen35_engine.h" in r.stdout and "src/adapters/tools/qwen35_engine.cpp" in r.stdout


def test_patched_engine_compiles_with_and_without_the_device_path(tmp_path):
    """Qwen35Engine with the patch: the translation unit compiles against the reference's headers with the device
    path switched on (gemm goes through gfx950::DeviceTensor) and, unchanged in meaning, with it switched off."""
    os.makedirs(tmp_path / "include" / "oil")
    os.makedirs(tmp_path / "src" / "adapters" / "tools")
    shutil.copy(os.path.join(REF, "include", "oil", "qwen35_engine.h"), tmp_path / "include" / "oil")
    shutil.copy(os.path.join(REF, "src", "adapters", "tools", "qwen35_engine.cpp"), tmp_path / "src" / "adapters" / "tools")
    subprocess.run(["patch", "-s", "-p1", "-d", str(tmp_path), "-i", ENGINE_PATCH], check=True)
    src = str(tmp_path / "src" / "adapters" / "tools" / "qwen35_engine.cpp")
    inc = [f"-I{tmp_path}/include", f"-I{REF}/include", f"-I{ROOT}/include"]
    for flags in (["-DOIL_USE_HIP_GFX950"], []):
        r = subprocess.run(["g++", "-std=c++20", "-fsyntax-only", "-w"] + flags + inc + [src], capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-4000:]
    text = open(src).read()
    assert "gfx950_gemm(t, X, Y, B)" in text and "decode_block(*reader_, bid, 256, sc)" in text   # both paths are there

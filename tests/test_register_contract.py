"""The register contract of the GEMM kernels whose accumulators are numbered by hand, read back from the BUILT library
(no GPU): the AMDGPU metadata notes of every code object inside libmi355_int8.so say how many registers each kernel
was given and how many the compiler spilled.  A kernel that spills, or that leaves the two-waves-per-SIMD budget,
would add into registers the compiler also uses, with wrong sums and no error at run time; the Makefile stops the
build on the compiler's own remarks, and this test holds the library that was actually built to the same contract.
A spilled scalar counts too: the compiler brings it back with a vector instruction, and a memory instruction inside
an asm statement would read it before it is valid."""
import os
import re
import struct
import subprocess
import sys
import tempfile

import pytest
import yaml

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "mojo-linuxperiments_amd", "libmi355_int8.so")
LLVM = "/opt/rocm/llvm/bin"
MAGIC = b"__CLANG_OFFLOAD_BUNDLE__"


def code_objects(lib):
    """The gfx950 code objects of every offload bundle in the library's .hip_fatbin section."""
    with tempfile.TemporaryDirectory() as tmp:
        fat = os.path.join(tmp, "fatbin")
        subprocess.check_call([os.path.join(LLVM, "llvm-objcopy"), "--dump-section", ".hip_fatbin=" + fat, lib,
                               os.path.join(tmp, "copy.so")])
        data = open(fat, "rb").read()
    out, at = [], data.find(MAGIC)
    while at >= 0:
        n = struct.unpack_from("<Q", data, at + len(MAGIC))[0]
        off = at + len(MAGIC) + 8
        for _ in range(n):
            o, size, tl = struct.unpack_from("<QQQ", data, off)
            off += 24
            triple = data[off:off + tl].decode()
            off += tl
            if "gfx950" in triple and size:
                out.append(data[at + o:at + o + size])
        at = data.find(MAGIC, at + len(MAGIC))
    return out


def kernel_notes(lib):
    """{mangled kernel name: {field: int}} over all code objects."""
    kernels = {}
    with tempfile.TemporaryDirectory() as tmp:
        for i, co in enumerate(code_objects(lib)):
            path = os.path.join(tmp, "co%d" % i)
            open(path, "wb").write(co)
            text = subprocess.run([os.path.join(LLVM, "llvm-readelf"), "--notes", path], capture_output=True, text=True,
                                  check=True).stdout
            # the metadata note is a YAML document between "---" and "..."
            for doc in re.findall(r"^\s*---\n(.*?)^\s*\.\.\.", text, flags=re.S | re.M):
                for k in (yaml.safe_load(doc) or {}).get("amdhsa.kernels", []):
                    kernels[k[".name"]] = {key.lstrip("."): val for key, val in k.items() if isinstance(val, int)}
    return kernels


@pytest.fixture(scope="module")
def notes():
    if not os.path.exists(LIB):
        pytest.skip("libmi355_int8.so is not built")
    if not all(os.path.exists(os.path.join(LLVM, t)) for t in ("llvm-objcopy", "llvm-readelf")):
        pytest.skip("llvm-objcopy / llvm-readelf not found under " + LLVM)
    return kernel_notes(LIB)


def test_the_library_holds_gfx950_kernels(notes):
    assert len(notes) > 50 and any("k_w8a8_list" in k for k in notes)


def test_batched_gemm_keeps_its_128_accumulators_to_itself(notes):
    mine = {k: v for k, v in notes.items() if "k_w8a8_list" in k}
    assert len(mine) == 2   # dequantized and int32 form
    for name, f in mine.items():
        # v0..v103 for the compiler, v104..v255 named by hand: the wave's count is the full 256 (two waves per SIMD),
        # no accumulation register, nothing in scratch, no vector and no scalar register spilled
        assert f["vgpr_count"] == 256 and f["agpr_count"] == 0, (name, f)
        assert f["vgpr_spill_count"] == 0 and f["sgpr_spill_count"] == 0 and f["private_segment_fixed_size"] == 0, (name, f)
        assert f["max_flat_workgroup_size"] == 512, (name, f)


def test_eight_wave_gemm_keeps_its_192_accumulation_registers_to_itself(notes):
    mine = {k: v for k, v in notes.items() if "k_w8a8_pair" in k}
    assert len(mine) == 4   # 8 x 6 and 4 x 8 tiles, dequantized and int32
    for name, f in mine.items():
        # a0..a191 named by hand; at most 64 ordinary registers beside them, none spilled (an ordinary register
        # spilled into an accumulation register would be overwritten by the matrix instructions)
        assert f["agpr_count"] == 192 and f["vgpr_count"] <= 256 and f["vgpr_count"] - f["agpr_count"] <= 64, (name, f)
        assert f["vgpr_spill_count"] == 0 and f["sgpr_spill_count"] == 0 and f["private_segment_fixed_size"] == 0, (name, f)
        assert f["max_flat_workgroup_size"] == 512, (name, f)


def test_no_kernel_with_memory_instructions_in_asm_spills_a_scalar(notes):
    for name, f in notes.items():
        if any(k in name for k in ("k_w8a8_tiled", "k_w8a8_pair", "k_w8a8_list")):
            assert f["sgpr_spill_count"] == 0, (name, f)


# ---- the batched GEMM's operand fragments: written by LDS reads behind the compiler's back, never to be copied

CHECK = os.path.join(ROOT, "mojo-linuxperiments_amd", "csrc", "check_fragment_registers.py")
ASM = os.path.join(ROOT, "mojo-linuxperiments_amd", "csrc", "gemm_list.s")

FAKE = """\
k_fake_list: ; @k_fake_list
\tds_read_b128 v[0:3], v70
\tds_read_b128 v[4:7], v70 offset:2048
\tv_mfma_i32_16x16x64_i8 v[128:131], v[4:7], v[0:3], v[128:131]
%s
\ts_endpgm
.Lfunc_end0:
"""


def run_check(path, *args):
    return subprocess.run([sys.executable, CHECK, path, *args], capture_output=True, text=True)


def test_fragment_check_passes_on_the_built_kernel():
    if not os.path.exists(ASM):
        pytest.skip("gemm_list.s is written by the build (make -C mojo-linuxperiments_amd/csrc)")
    out = run_check(ASM, "k_w8a8_list", "16")
    assert out.returncode == 0, out.stderr[-2000:]
    assert "2 kernel(s)" in out.stdout


def test_fragment_check_fails_on_a_copied_fragment_and_on_a_fragment_that_moved(tmp_path):
    good = tmp_path / "good.s"
    good.write_text(FAKE % "\tv_mov_b32_e32 v9, v64")            # a move INTO a dead fragment register is fine
    assert run_check(str(good), "k_fake_list", "2").returncode == 0
    copied = tmp_path / "copied.s"
    copied.write_text(FAKE % "\tv_mov_b32_e32 v9, v5")           # a move OUT of one is not
    out = run_check(str(copied), "k_fake_list", "2")
    assert out.returncode != 0 and "copies fragment register v5" in out.stderr
    moved = tmp_path / "moved.s"
    moved.write_text(FAKE % "\tds_read_b128 v[8:11], v70")       # a third range where two are expected
    out = run_check(str(moved), "k_fake_list", "2")
    assert out.returncode != 0 and "3 distinct register ranges" in out.stderr
    assert run_check(str(good), "k_absent").returncode != 0

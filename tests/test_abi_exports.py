"""The shared library loads on a machine without a GPU and exports every
symbol the header declares (no compute call is made here)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355_int8.h")
LIB = os.path.join(ROOT, "mojo-linuxperiments_amd", "libmi355_int8.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"MI_API\s+[\w\s\*]+?\b(mi_\w+)\s*\(", text)))


def test_header_declares_the_expected_families():
    names = declared_symbols()
    assert len(names) >= 50
    for fam in ("mi_arena_", "mi_stream_pool_", "mi_gate_", "mi_fwht_", "mi_w8a8_", "mi_gqa_", "mi_moe_"):
        assert any(n.startswith(fam) for n in names), fam


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "build first: python -c 'import __graft_entry__ as g; g.build()'"
    lib = ctypes.CDLL(LIB)
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_covers_every_declared_symbol(mi):
    assert sorted(mi.SIGNATURES) == declared_symbols()


def test_status_strings_and_argument_checks_without_gpu(mi):
    lib = mi.lib
    assert lib.mi_abi_version() == 1
    assert lib.mi_status_string(0) == b"ok"
    assert lib.mi_status_string(mi.EINVAL) == b"invalid argument"
    # pure argument validation happens before any HIP call
    assert lib.mi_fwht_quant_f32_i8(None, None, None, 1, 128, 128, None) == mi.EINVAL
    assert lib.mi_w8a8_gemm_i32(None, None, None, 1, 16, 128, None) == mi.EINVAL
    assert lib.mi_arena_alloc(None, 16) is None
    assert lib.mi_arena_mark(None) == mi.EINVAL
    assert lib.mi_stream_pool_begin(None) == mi.EINVAL
    assert lib.mi_w8a8_linear_workspace_bytes(32, 4096, 4096) >= 32 * 4096 + 32 * 4
    assert lib.mi_gqa_decode_workspace_bytes(16, 32, 8, 64, 4096) == mi.EINVAL      # head_dim must be 128
    assert lib.mi_gqa_decode_workspace_bytes(16, 32, 6, 128, 4096) == mi.EINVAL     # Hq % Hkv


def test_attention_workspace_bound_covers_every_shorter_length(mi):
    """A workspace sized for the capacity of a cache must serve every decode step: the split plan is not monotone
    in the length (a shorter sequence may be cut into more, shorter spans), the size query is."""
    lib = mi.lib
    for rows, hkv in ((128, 8), (64, 8), (32, 8), (16, 8), (8, 8), (1, 1), (3, 1)):
        B = rows // hkv if rows >= hkv else rows
        for t_cap in (48, 1000, 2048, 4096, 16384):
            cap = lib.mi_gqa_decode_workspace_bytes(B, 4 * hkv, hkv, 128, t_cap)
            assert cap > 0
            prev = 0
            for t in list(range(1, min(t_cap, 600))) + list(range(600, t_cap + 1, 37)) + [t_cap]:
                need = lib.mi_gqa_decode_workspace_bytes(B, 4 * hkv, hkv, 128, t)
                assert prev <= need <= cap, (rows, t_cap, t)
                prev = need


MOJO = os.path.join(ROOT, "mojo-linuxperiments_amd", "host", "mi355.mojo")


def test_mojo_host_surface_binds_only_exported_symbols_and_all_of_them():
    """host/mi355.mojo cannot be compiled here (no Mojo toolchain); what can be held to the library is its symbol
    list: every name it looks up is exported, and it binds every entry point the header declares."""
    text = open(MOJO).read()
    names = set(re.findall(r'\("(mi_\w+)"\)', text))
    assert len(names) >= 60
    lib = ctypes.CDLL(LIB)
    missing = sorted(n for n in names if not hasattr(lib, n))
    assert not missing, missing
    unbound = sorted(set(declared_symbols()) - names)
    assert not unbound, unbound

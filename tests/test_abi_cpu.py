"""CPU-only checks of the C-ABI library: it loads, exports every symbol the header declares, the
ctypes table matches the header, and argument validation fails loudly without touching a GPU."""
import ctypes as C
import os
import re

import pytest

from msa_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "msa_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(msa_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    lib = _lib.load()
    names = _declared()
    assert len(names) >= 16
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names
    assert lib.msa_abi_version() == 1


def test_header_arity_matches_ctypes_table():
    text = open(os.path.join(ROOT, "include", "msa_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    for name, (_, args) in _lib.SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % name, text, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else len(params.split(","))
        assert n == len(args), f"{name}: header has {n} parameters, ctypes table {len(args)}"


def test_validation_errors_without_gpu():
    lib = _lib.load()
    # wrong head dim
    rc = lib.msa_pool_chunks(None, None, None, 0, 10, 8, 64, None, None, None, 1, None, None, None, 0, 0, 0, None,
                             None, None, None)
    assert rc == -1 and b"head dim" in lib.msa_last_error()
    # null bank
    rc = lib.msa_route_topk(None, 0, None, None, 1, 1, 32, 0, 1.0, 16, C.c_void_p(8), C.c_void_p(8), None, None, 0,
                            None)
    assert rc == -1 and b"null bank" in lib.msa_last_error()
    rc = lib.msa_route_topk(None, 0, None, None, 1, 1, 32, 0, 1.0, 65, C.c_void_p(8), C.c_void_p(8), None, None, 0,
                            None)
    assert rc == -1 and b"topk" in lib.msa_last_error()
    # bank tables that do not add up are rejected before any device call
    off = (C.c_int32 * 3)(0, 2, 5)
    gid = (C.c_int64 * 2)(7, 9)
    h = C.c_void_p()
    rc = lib.msa_bank_create(C.byref(h), 1, 6, 8, 128, 0, C.addressof(off), C.addressof(gid), 2)
    assert rc == -1 and b"doc_chunk_off" in lib.msa_last_error()
    assert lib.msa_route_workspace_bytes(16, 128, 32, 8, 128, 1000, 50, 16) > 16 * 128 * 1024 * 2
    assert lib.msa_attn_workspace_bytes(4, 32, 8, 128, 1000) > 0
    # many query rows: one pass over the keys, so the workspace stays linear in the rows
    assert lib.msa_attn_workspace_bytes(65536, 32, 8, 128, 4400) < 2 * 65536 * 32 * 130 * 4
    with pytest.raises(TypeError):
        import torch
        _lib.dtype_code(torch.float16)


def test_product_does_not_import_oracle():
    """Nothing under msa_amd/ may reach into oracle/."""
    pkg = os.path.join(ROOT, "msa_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.replace("ORACLE", ""), f"{f} mentions the oracle"


@pytest.mark.parametrize("tiles_m,tiles_n,grid,copy_wg,pool_n", [
    (8, 6271, 256, 1, 783), (8, 6271, 256, 0, 783), (8, 6271, 256, 1, 0),      # the 100M-token bank, B = 16 x 128
    (16, 628, 256, 0, 78), (16, 628, 256, 1, 0),                                # the 10M-token bank, B = 32 x 128
    (1, 40, 256, 0, 0), (2, 3, 16, 1, 0), (3, 100, 64, 1, 12), (11, 37, 256, 0, 4), (11, 37, 24, 1, 18),
    (20, 999, 248, 1, 124), (256, 628, 256, 0, 78), (9, 5, 1024, 1, 0), (5, 1, 16, 0, 0), (7, 200, 16, 1, 25),
])
def test_scan_tile_order_covers_every_tile_once(tiles_m, tiles_n, grid, copy_wg, pool_n):
    """The persistent scan's tile order (fixed shares per XCD walked by an incremental cursor, then the pool):
    every tile exactly once, for grids with and without the copying workgroup and with and without a pool."""
    lib = _lib.load()
    visits = (C.c_int32 * (tiles_m * tiles_n))()
    rc = lib.msa_diag_scan_walk(tiles_m, tiles_n, grid, copy_wg, pool_n, C.addressof(visits))
    assert rc == 0, lib.msa_last_error()
    v = list(visits)
    assert min(v) == 1 and max(v) == 1, f"{v.count(0)} tiles unvisited, {sum(1 for x in v if x > 1)} visited twice"


def test_tile_pool_switch_is_exported():
    lib = _lib.load()
    assert lib.msa_route_set_tile_pool(0) == 0
    assert lib.msa_route_set_tile_pool(1) == 0


def test_build_guard_flags_compiler_code_in_the_asm_statements_registers():
    """The build checks the device assembly of the hand-scheduled scan: code the compiler generated for it (outside
    the inline-asm regions) must stay below v128, leave the accumulation registers alone and use no scratch."""
    from msa_amd import build as B
    ok = """
_ZN12_GLOBAL__N_118score_scan4_kernelILb1EEEvPKt:
	v_add_u32_e32 v5, v4, v3
	;;#ASMSTART
	v_mfma_f32_32x32x16_bf16 a[0:15], v[128:131], v[144:147], a[0:15]
	;;#ASMEND
	s_endpgm
"""
    assert B.check_kernel_contracts(ok, "score_scan4_kernel", max_compiler_vgpr=127, no_agpr=True) == []
    bad = ok.replace("v_add_u32_e32 v5, v4, v3", "v_accvgpr_write_b32 a3, v7\n\tv_mov_b32_e32 v130, v2\n\tscratch_store_dword off, v1, s32")
    problems = B.check_kernel_contracts(bad, "score_scan4_kernel", max_compiler_vgpr=127, no_agpr=True)
    assert len(problems) == 3, problems
    assert B.check_kernel_contracts(ok, "no_such_kernel") != []


def test_build_guard_fails_on_a_forced_spill():
    """With the compiler's share of the scan kernel's registers cut to 24 the kernel spills, and the check that
    build() runs on the device assembly reports it (this compiles route_score.hip once: about 15 s)."""
    from msa_amd import build as B
    src = open(os.path.join(B.CSRC, "route_score.hip")).read()
    assert "constexpr int kScan4CompilerVgprs = 128;" in src
    tmp = os.path.join(B.CSRC, "_guard_probe.hip")            # beside the sources: it includes its neighbours
    try:
        open(tmp, "w").write(src.replace("constexpr int kScan4CompilerVgprs = 128;", "constexpr int kScan4CompilerVgprs = 24;"))
        asm = B._device_asm(tmp)
    finally:
        if os.path.exists(tmp):
            os.remove(tmp)
    problems = B.check_kernel_contracts(asm, "score_scan4_kernel", max_compiler_vgpr=127, no_agpr=True)
    assert problems, "a spilling build passed the check"
    assert any("spill" in p or "scratch" in p or "private_segment" in p or "accumulation" in p for p in problems), problems[:5]


@pytest.mark.parametrize("gen", ["gen_scan_asm.py", "gen_flash_asm.py"])
def test_generated_asm_includes_are_what_their_generators_emit(gen):
    """The committed scan_asm.inc / flash_asm.inc are the generators' output (the build refuses a stale one too)."""
    import subprocess
    import sys
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "msa_amd", "csrc")
    assert subprocess.run([sys.executable, os.path.join(csrc, gen), "--check"]).returncode == 0


def test_build_guard_covers_the_wide_flash_kernel():
    from msa_amd import build
    names = [k for k, _ in build.CONTRACTS["flash_attn.hip"]]
    assert "flash_wide_kernel" in names and "flash_attn_kernel" in names
    rules = dict(build.CONTRACTS["flash_attn.hip"])["flash_wide_kernel"]
    assert rules == {"max_compiler_vgpr": 55, "no_agpr": True}

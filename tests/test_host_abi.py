"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol the header
declares, and rejects bad shapes/handles before touching a device."""
import ctypes as C
import os
import re

import pytest

from openagents_amd import _ffi, backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return _ffi.load()


def header_functions():
    text = open(os.path.join(ROOT, "include", "psn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(psn_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    names = header_functions()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/psn.h but not exported"
        assert n in _ffi.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_ffi.SIGNATURES) == names
    assert lib.psn_abi_version() == 1


def test_block_geometry(lib):
    assert [lib.psn_block_bytes(t) for t in (_ffi.Q8_0, _ffi.Q4_0, _ffi.Q4_K, _ffi.Q6_K, _ffi.Q8_K)] == [34, 18, 144, 210, 292]
    assert [lib.psn_block_elems(t) for t in (_ffi.Q8_0, _ffi.Q4_0, _ffi.Q4_K, _ffi.Q6_K)] == [32, 32, 256, 256]
    assert backend.row_bytes(_ffi.Q4_0, 4096) == 2304
    assert backend.row_bytes(_ffi.Q4_K, 14336) == 8064
    assert backend.row_bytes(_ffi.Q6_K, 4096) == 3360
    with pytest.raises(backend.PsnError) as e:
        backend.row_bytes(_ffi.Q4_K, 4096 + 32)
    assert e.value.code == _ffi.E_SHAPE and "multiple" in str(e.value)
    with pytest.raises(backend.PsnError) as e:
        backend.row_bytes(99, 4096)
    assert e.value.code == _ffi.E_UNSUPPORTED


def test_activation_layout(lib):
    li = backend.actq_layout(_ffi.Q8_0, 4096, 1)
    assert (li.off_qs, li.off_d, li.off_s) == (0, 4096, 4096 + 512) and li.bytes == 4096 + 512 + 512
    li = backend.actq_layout(_ffi.Q8_K, 14336, 8)
    assert li.off_d == 8 * 14336 and li.off_d % 256 == 0 and li.off_s % 256 == 0
    assert li.bytes >= li.off_s + 8 * (14336 // 16) * 2
    assert backend.act_type_for(_ffi.Q4_0) == _ffi.Q8_0 and backend.act_type_for(_ffi.Q6_K) == _ffi.Q8_K
    for bad in (0, 9):
        with pytest.raises(backend.PsnError) as e:
            backend.actq_layout(_ffi.Q8_0, 4096, bad)
        assert e.value.code == _ffi.E_SHAPE
    with pytest.raises(backend.PsnError) as e:
        backend.actq_layout(_ffi.Q4_0, 4096, 1)
    assert e.value.code == _ffi.E_UNSUPPORTED


def test_matvec_plan_is_host_arithmetic(lib):
    for qt in (_ffi.Q4_0, _ffi.Q8_0, _ffi.Q4_K, _ffi.Q5_K, _ffi.Q6_K):
        for (n, k) in ((4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (128256, 4096), (1, 256)):
            for batch in range(1, 9):
                for scheme in (_ffi.ACT_F32, _ffi.ACT_Q8):
                    p = backend.matvec_plan(qt, scheme, n, k, batch)
                    assert p.lanes_per_row in (8, 16, 32, 64) and p.rows_in_flight == 1
                    assert p.batch_tile >= batch and p.batch_tile in (1, 2, 4, 8)
                    assert 1 <= p.blocks <= 256 * 16
                    assert p.threads in (256, 512) or (p.stream and not p.mfma and p.threads in (320, 384, 448))
                    assert p.mfma in (0, 1, 2, 4, 8) and (p.mfma == 0 or (batch >= 2 and scheme == _ffi.ACT_Q8 and qt in (_ffi.Q4_K, _ffi.Q5_K)))
    for args, code in (((_ffi.Q4_0, 1, 0, 4096, 1), _ffi.E_SHAPE), ((_ffi.Q4_0, 1, 16, 4096 + 32, 1), _ffi.E_SHAPE),
                       ((_ffi.Q4_0, 1, 16, 4096, 9), _ffi.E_SHAPE), ((_ffi.Q8_K, 1, 16, 4096, 1), _ffi.E_UNSUPPORTED),
                       ((_ffi.Q4_0, 5, 16, 4096, 1), _ffi.E_UNSUPPORTED)):
        with pytest.raises(backend.PsnError) as e:
            backend.matvec_plan(*args)
        assert e.value.code == code, args


def test_matvec_plans_are_consistent_over_many_shapes(lib):
    """Host arithmetic only: every plan the library returns over a grid of shapes and batches is one its own
    kernels accept (thread counts, slice arithmetic of the MFMA kernels, enough workgroups for one-unit waves)."""
    for qt in (_ffi.Q4_0, _ffi.Q8_0, _ffi.Q4_K, _ffi.Q5_K, _ffi.Q6_K):
        for k in (256, 512, 768, 1024, 2048, 2304, 4096, 5120, 8192, 11008, 14336, 16384, 28672):
            for n in (1, 16, 17, 48, 1000, 1024, 4096, 14336, 128256):
                for batch in (1, 2, 3, 5, 8):
                    for x_is_f32 in (False, True):
                        p = backend.matvec_plan(qt, _ffi.ACT_Q8, n, k, batch, 256, x_is_f32)
                        assert 1 <= p.blocks <= 1 << 20, p.as_dict()
                        # four or eight waves; the batch-1 streaming kernels also take five to seven
                        assert p.threads in (256, 512) or (p.stream and not p.mfma and p.threads in (320, 384, 448)), p.as_dict()
                        if p.mfma:
                            c, waves = k // 256, p.threads // 64
                            assert qt in (_ffi.Q4_K, _ffi.Q5_K) and batch >= 2 and n % 16 == 0, p.as_dict()
                            assert p.mfma in (1, 2, 4, 8) and p.mfma <= waves and c % p.mfma == 0 and c // p.mfma <= 8, p.as_dict()
                            assert p.stage_lds == 1 and p.stream == 1, p.as_dict()
                            if c // p.mfma > 4:
                                assert p.blocks * (waves // p.mfma) >= n // 16, p.as_dict()      # one wave per unit
                            lds = c * 160 + waves * 1024 + waves * (9 if qt == _ffi.Q4_K else 11) * 1024
                            assert lds <= 160 * 1024, p.as_dict()
                        elif p.stream:
                            assert batch == 1 and p.stage_lds in (1, 2) and k // 256 <= p.lanes_per_row, p.as_dict()
                            npass = n // (64 // p.lanes_per_row)
                            if 4 * 256 < npass <= 8 * 256 and p.threads < 512:
                                # one pass per wave, one workgroup on every compute unit
                                assert p.blocks == 256 and p.blocks * (p.threads // 64) >= npass, p.as_dict()
    # Llama-3-8B's fused q/k/v projection: 6144 rows of sixteen chunks, four rows a pass -> 1536 passes = 256 x 6 waves
    p = backend.matvec_plan(_ffi.Q4_0, _ffi.ACT_Q8, 6144, 4096, 1, 256, True)
    assert (p.stream > 0, p.threads, p.blocks) == (True, 384, 256), p.as_dict()


def test_swiglu_fused_launch_check_is_host_arithmetic(lib):
    """psn_qmatvec_norm_swiglu_check: which gate|up shapes the SwiGLU-fused launch serves, without a device."""
    chk = lambda qt, n, k: int(lib.psn_qmatvec_norm_swiglu_check(qt, n, k, 256))
    for qt in (_ffi.Q4_0, _ffi.Q8_0, _ffi.Q4_K, _ffi.Q5_K, _ffi.Q6_K):
        assert chk(qt, 14336, 4096) == 0 and chk(qt, 1024, 2048) == 0
        assert chk(qt, 4096, 14336) == _ffi.E_UNSUPPORTED              # rows longer than the fused staging holds
        assert chk(qt, 1026, 4096) == _ffi.E_UNSUPPORTED               # not whole passes
        assert chk(qt, 0, 4096) == _ffi.E_SHAPE and chk(qt, 1024, 4100) == _ffi.E_SHAPE
    assert chk(_ffi.Q6_K, 1024, 2304) == _ffi.E_UNSUPPORTED            # 210-byte blocks: rows of whole 16-byte words only
    assert chk(_ffi.Q8_K, 1024, 4096) != 0                             # not a weight format


def test_prefill_plans_are_consistent_over_many_shapes(lib):
    """Host arithmetic only: every prefill plan over a grid of shapes is one psn_qmatmul_prefill_tiled accepts --
    a known tile, a family the format has, a K split that leaves whole chunks per range and an atomically addable Y."""
    tiles = {(64, 64), (64, 128), (128, 128), (128, 256), (256, 128), (256, 256)}
    for qt in (_ffi.Q4_0, _ffi.Q8_0, _ffi.Q4_K, _ffi.Q5_K, _ffi.Q6_K):
        for k in (256, 512, 1024, 2048, 2304, 4096, 5120, 8192, 11008, 14336):
            for n in (1, 17, 64, 130, 1000, 1024, 4096, 6144, 14336):
                for m in (1, 7, 64, 65, 128, 200, 512, 777, 2048, 4096):
                    tm, tn, sp, wv = backend.prefill_plan(m, n, k, 256, qt)
                    tag = (qt, m, n, k, tm, tn, sp, wv)
                    assert (tm, tn) in tiles and sp in (1, 2, 4, 8), tag
                    if sp > 1:
                        assert (m * n) % 4 == 0 and k // 256 >= 2 * sp, tag
                    if m <= 64 and (qt != _ffi.Q6_K or k % 2048 == 0):
                        assert wv == 64 and (tm, tn) == (64, 64), tag           # the weight-streaming kernel
                    else:
                        assert wv != 64, tag
                    if wv == 128:
                        assert m > 64 and tn == 256 and tm in (128, 256) and sp <= 4, tag
                    elif wv == 32:
                        assert qt in (_ffi.Q4_0, _ffi.Q8_0) and (tm, tn) == (256, 256), tag
                    elif wv == 16:
                        assert (tm, tn) in {(64, 64), (64, 128), (128, 128), (128, 256)}, tag
                        assert qt in (_ffi.Q4_0, _ffi.Q8_0) or (qt != _ffi.Q6_K and (tm, tn) == (128, 256)), tag
                    else:
                        assert wv in (4, 64), tag


def test_null_handles_are_rejected_without_a_device(lib):
    assert lib.psn_stream_sync(None) == _ffi.E_INVALID_ARG
    assert lib.psn_buf_free(None) == _ffi.E_INVALID_ARG
    assert lib.psn_module_unload(None) == _ffi.E_INVALID_ARG
    assert lib.psn_ctx_destroy(None) == _ffi.E_INVALID_ARG
    assert lib.psn_qmatvec(None, None, _ffi.Q4_0, 0, 1, None, None, None, 16, 4096, 1) == _ffi.E_INVALID_ARG
    assert b"null" in lib.psn_last_error()
    assert lib.psn_qmatvec(None, None, _ffi.Q4_0, 7, 1, None, None, None, 16, 4096, 1) == _ffi.E_UNSUPPORTED
    h = C.c_void_p()
    assert lib.psn_buf_alloc(None, 16, C.byref(h)) == _ffi.E_INVALID_ARG and not h.value
    assert lib.psn_module_load(None, None, 0, C.byref(h)) == _ffi.E_INVALID_ARG
    assert lib.psn_error_name(-4) == b"PSN_E_NO_DEVICE"


def test_context_creation_fails_loudly_without_gfx950(lib):
    h = C.c_void_p()
    rc = lib.psn_ctx_create(0, C.byref(h))
    if rc == 0:                      # running on a GPU box: nothing to assert about absence
        assert lib.psn_ctx_destroy(h) == 0
        return
    assert rc == _ffi.E_NO_DEVICE and not h.value
    assert lib.psn_last_error()
    with pytest.raises(backend.PsnError):
        backend.HipBackend(0)


def test_missing_library_is_an_error_not_a_fallback(monkeypatch):
    monkeypatch.setattr(_ffi, "_lib", None)
    monkeypatch.setattr(_ffi, "LIB_PATH", "/nonexistent/libpsn_hip.so")
    with pytest.raises(_ffi.LibraryMissing):
        _ffi.load()


def test_integration_doc_binding_lists_every_entry_point():
    """The Rust `-sys` text a maintainer would paste must not drift from the header."""
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    rust = set(re.findall(r"pub fn (psn_[a-z0-9_]+)\(", doc))
    assert rust == set(header_functions())


def test_static_scratch_is_exported_by_the_device_image():
    """The no-allocation entry point finds its scratch with hipGetSymbolAddress, which looks the
    registered name up among the symbols the gfx950 image EXPORTS; a file-local symbol there makes the
    runtime abort.  Checked on the built object, no GPU needed."""
    import shutil
    import subprocess
    import tempfile
    obj = os.path.join(ROOT, "openagents_amd", "lib", "psn_noalloc.o")
    bundler, readelf = "/opt/rocm/llvm/bin/clang-offload-bundler", "/opt/rocm/llvm/bin/llvm-readelf"
    if not (os.path.exists(obj) and os.path.exists(bundler) and os.path.exists(readelf) and shutil.which("objcopy")):
        pytest.skip("built object or LLVM binutils not present")
    with tempfile.TemporaryDirectory() as d:
        fat, elf = os.path.join(d, "fat.bin"), os.path.join(d, "dev.elf")
        subprocess.check_call(["objcopy", "-O", "binary", "--only-section=.hip_fatbin", obj, fat])
        subprocess.check_call([bundler, "--unbundle", "--type=o", f"--input={fat}", "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", f"--output={elf}"])
        syms = subprocess.check_output([readelf, "--dyn-syms", elf], text=True)
    rows = [ln.split() for ln in syms.splitlines() if ln.strip().endswith("scratch")]
    assert rows, syms
    assert all(r[3] == "OBJECT" and r[4] == "GLOBAL" and int(r[2]) == 1 << 20 for r in rows), rows


def _kernel_resources():
    """name -> (vgpr spills, sgpr spills, scratch bytes per lane) for every kernel of every built code object,
    read from the code objects' own metadata notes."""
    import glob
    import subprocess
    import tempfile
    bundler, readelf = "/opt/rocm/llvm/bin/clang-offload-bundler", "/opt/rocm/llvm/bin/llvm-readelf"
    objs = sorted(glob.glob(os.path.join(ROOT, "openagents_amd", "lib", "*.gfx950.hsaco")))
    if not objs or not (os.path.exists(bundler) and os.path.exists(readelf)):
        pytest.skip("built code objects or LLVM binutils not present")
    out = {}
    with tempfile.TemporaryDirectory() as d:
        for path in objs:
            elf = os.path.join(d, os.path.basename(path) + ".elf")
            subprocess.check_call([bundler, "--unbundle", "--type=o", f"--input={path}", "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", f"--output={elf}"])
            notes = subprocess.check_output([readelf, "--notes", elf], text=True)
            for blk in notes.split("- .agpr_count:")[1:]:
                get = lambda key: re.search(r"\." + key + r":\s+(\S+)", blk).group(1)
                out[get("name")] = (int(get("vgpr_spill_count")), int(get("sgpr_spill_count")), int(get("private_segment_fixed_size")))
    return out


def test_no_kernel_spills_registers_or_uses_scratch():
    """Every kernel a planner can return (and every other kernel of the library) keeps its working set in
    registers: a spilled register or a scratch copy of the kernel arguments costs memory round trips in the
    middle of a stream and has gone unnoticed before."""
    res = _kernel_resources()
    assert len(res) > 300
    for family in ("psn_mvs_q4_0_q8_g16_xf_s2", "psn_mvs_q6_K_q8_g16_lds_s1", "psn_prefill_q4_0_skinny", "psn_prefill_q8_0_m128_n256_ws",
                   "psn_prefill_q4_0_m256_n256", "psn_attn_partial_rope", "psn_mv_q4_K_q8_g16_r1_b8_lds"):
        assert family in res, family
    bad = {k: v for k, v in res.items() if v != (0, 0, 0)}
    assert not bad, bad


def test_prefill_plans_take_the_dense_family_only_for_large_m():
    """Host arithmetic: from a few thousand rows of X on every format is dequantized once and multiplied as
    fp16 (family 128, 256 x 256 or 128 x 256 tiles); 64 rows and fewer never are."""
    for qt in (_ffi.Q4_0, _ffi.Q8_0, _ffi.Q4_K, _ffi.Q5_K, _ffi.Q6_K):
        for n, k in ((14336, 4096), (4096, 14336)):
            tm, tn, sp, wv = backend.prefill_plan(4096, n, k, 256, qt)
            assert tm in (128, 256) and (tn, wv) == (256, 128) and sp in (1, 2, 4), (qt, n, k)
            for m in (1, 16, 64):
                assert backend.prefill_plan(m, n, k, 256, qt)[3] == 64     # 64 rows and fewer: the weight-streaming kernel
    assert backend.prefill_plan(64, 4096, 4096 + 256, 256, _ffi.Q6_K)[3] == 4   # Q6_K rows that are not whole 16-byte words
    lib = _ffi.load()
    assert lib.psn_error_name(lib.psn_prefill_reserve(None, 4096, 4096)) == b"PSN_E_INVALID_ARG"

"""CPU-side checks of the boundary: the shared library loads without a GPU and exports
every symbol that include/tract_rocm.h declares; the host mirror refuses to run without
the device instead of falling back."""
import os
import re
import subprocess

import pytest

from tests.conftest import ROOT


def _header_symbols():
    text = open(os.path.join(ROOT, "include", "tract_rocm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(trocm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from tract_amd import _lib
    lib = _lib.load()
    names = _header_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), f"{n} declared in tract_rocm.h but not exported"
    assert set(_lib.SIGNATURES) == set(names)
    out = subprocess.check_output(["nm", "-D", "--defined-only", _lib.LIB_PATH], text=True)
    exported = set(re.findall(r" T (trocm_[a-z0-9_]+)", out))
    assert exported == set(names)


def test_rust_binding_matches_header():
    """The Rust `extern "C"` block a maintainer pastes into rocm/src/ffi.rs declares every entry point of the
    header with the same arguments: the copy in the integration notes is the generator's output for today's header."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("gen_rust_ffi", os.path.join(ROOT, "include", "gen_rust_ffi.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    header = open(os.path.join(ROOT, "include", "tract_rocm.h")).read()
    decls = gen.declarations(header)
    assert [d[0] for d in decls] == sorted(set(d[0] for d in decls), key=[d[0] for d in decls].index)   # no duplicates
    assert sorted(d[0] for d in decls) == _header_symbols()
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = re.search(r'extern "C" \{\n.*?\n\}', doc, flags=re.S).group(0)
    assert block == gen.rust_block(header)
    # argument counts, independently of the generator's type mapping
    doc_fns = dict((m.group(1), m.group(2)) for m in re.finditer(r"pub fn (trocm_[a-z0-9_]+)\((.*?)\) ->", block))
    for name, _ret, params in decls:
        n_doc = 0 if not doc_fns[name].strip() else doc_fns[name].count(":")
        assert n_doc == len(params), name
    # every opaque handle the block mentions is declared beside it
    for opaque in set(re.findall(r"\b(trocm_[a-z0-9_]+)\b(?!\()", block)) - set(doc_fns):
        assert f"pub struct {opaque}" in doc, opaque


def test_header_is_plain_c():
    src = '#include "tract_rocm.h"\nint main(void){return (int)sizeof(trocm_dtype) == 0;}\n'
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), "-x", "c", "-",
                    "-fsyntax-only"], input=src, text=True, check=True)


def test_error_convention_without_device():
    import tract_amd
    from tract_amd import _lib
    lib = _lib.load()
    if lib.trocm_init(0) == 0:
        pytest.skip("GPU present")
    # KO + message, and no fallback path: the runtime cannot be created
    assert b"HIP device" in lib.trocm_last_error()
    with pytest.raises(tract_amd.TractRocmError):
        tract_amd.runtime_for_name("rocm")
    with pytest.raises(tract_amd.TractRocmError):
        tract_amd.runtime_for_name("cuda")
    # null pointers are reported, never dereferenced
    assert lib.trocm_kv_cache_len(None, None) == 1
    assert b"null pointer" in lib.trocm_last_error()


def test_no_kernel_spills_registers():
    """A kernel that spills to scratch still computes the right thing and runs several times
    slower (it happened twice while these kernels were written); the build records hipcc's
    per-kernel resource usage and this test reads it."""
    from tract_amd.build import resource_usage
    usage = resource_usage()
    assert len(usage) > 50
    spilling = {k: v for k, v in usage.items() if v.get("VGPRs Spill", 0) or v.get("SGPRs Spill", 0) or v.get("ScratchSize [bytes/lane]", 0)}
    assert not spilling, spilling
    # the kernels that must keep two waves per SIMD resident do
    for name, v in usage.items():
        if "sdpa_prefill_pp_kernel" in name:
            assert v["Occupancy [waves/SIMD]"] >= 2, (name, v)

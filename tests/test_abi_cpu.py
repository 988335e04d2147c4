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


def _load_generator():
    import importlib.util
    spec = importlib.util.spec_from_file_location("gen_rust_ffi", os.path.join(ROOT, "include", "gen_rust_ffi.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    return gen


def test_rust_binding_matches_header():
    """rust/tract-rocm/src/ffi.rs is the generator's output for today's header, and declares every entry point with
    the header's arguments."""
    gen = _load_generator()
    header = open(os.path.join(ROOT, "include", "tract_rocm.h")).read()
    decls = gen.declarations(header)
    assert [d[0] for d in decls] == sorted(set(d[0] for d in decls), key=[d[0] for d in decls].index)   # no duplicates
    assert sorted(d[0] for d in decls) == _header_symbols()
    ffi = open(os.path.join(ROOT, "rust", "tract-rocm", "src", "ffi.rs")).read()
    assert ffi == gen.rust_file(header), "rust/tract-rocm/src/ffi.rs is stale: run python include/gen_rust_ffi.py --write"
    block = re.search(r'extern "C" \{\n.*?\n\}', ffi, flags=re.S).group(0)
    # argument counts, independently of the generator's type mapping
    ffi_fns = dict((m.group(1), m.group(2)) for m in re.finditer(r"pub fn (trocm_[a-z0-9_]+)\((.*?)\) ->", block))
    for name, _ret, params in decls:
        n_ffi = 0 if not ffi_fns[name].strip() else ffi_fns[name].count(":")
        assert n_ffi == len(params), name
    # every opaque handle the block mentions is declared beside it, every enumerator of the header is a constant
    for opaque in set(re.findall(r"\b(trocm_[a-z0-9_]+)\b(?!\()", block)) - set(ffi_fns):
        assert f"pub struct {opaque}" in ffi, opaque
    for const, val in gen.enum_constants(header):
        assert f"pub const {const}: c_int = {val};" in ffi


def _rust_calls(text):
    """[(entry point, number of arguments)] of every `ffi::trocm_*( ... )` call in a Rust source text."""
    text = re.sub(r"//[^\n]*", "", text)
    out = []
    for m in re.finditer(r"ffi::(trocm_[a-z0-9_]+)\s*\(", text):
        depth, i, commas, any_arg = 1, m.end(), 0, False
        while depth:
            ch = text[i]
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
            elif ch == "," and depth == 1:
                commas += 1
            elif not ch.isspace() and depth >= 1:
                any_arg = True
            i += 1
        last = text[m.end():i - 1].rstrip()
        trailing = last.endswith(",")
        out.append((m.group(1), (commas + (0 if trailing else 1)) if any_arg else 0))
    return out


def test_rust_sources_call_the_abi_as_declared():
    """Every `ffi::trocm_*` call in rust/ names an entry point of the header and passes as many arguments as the
    header declares (the Rust is compile-unverified: this is the mechanical part of a compiler's check)."""
    gen = _load_generator()
    header = open(os.path.join(ROOT, "include", "tract_rocm.h")).read()
    arity = {name: len(params) for name, _ret, params in gen.declarations(header)}
    seen = set()
    n_files = 0
    for dirpath, _dirs, files in os.walk(os.path.join(ROOT, "rust")):
        for f in files:
            if not f.endswith(".rs") or f == "ffi.rs":
                continue
            n_files += 1
            path = os.path.join(dirpath, f)
            for name, n in _rust_calls(open(path).read()):
                assert name in arity, f"{path}: {name} is not declared in tract_rocm.h"
                assert n == arity[name], f"{path}: {name} called with {n} arguments, the header declares {arity[name]}"
                seen.add(name)
    assert n_files >= 10
    # the path's entry points are all reached from the Rust side
    for must in ("trocm_init", "trocm_copy_nd", "trocm_kv_append", "trocm_inplace_kv_sdpa_eval", "trocm_window_kv_sdpa_eval", "trocm_sdpa",
                 "trocm_kv_export", "trocm_kv_import_blocks", "trocm_kv_cache_clone", "trocm_kv_cache_truncate", "trocm_quantized_kv_sdpa_eval",
                 "trocm_kivi_cache_append", "trocm_kivi_cache_dequantize", "trocm_cast", "trocm_apply_rope", "trocm_rotate_half",
                 "trocm_sdpa_workspace_bytes", "trocm_sdpa_workspace_init", "trocm_malloc", "trocm_free", "trocm_h2d", "trocm_d2h"):
        assert must in seen, f"{must} is never called from rust/"


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

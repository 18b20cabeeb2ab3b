"""CPU tests of the run-time compiler path and its on-disk cache.

hiprtc compiles for gfx950 without a GPU being present, so everything except
loading the code object onto a device is exercised here.
"""
import json

import pytest

import kermac_amd as kermac
from kermac_amd.module_cache import module_cache as mc
from kermac_amd.module_cache.code_object_store import CodeObjectStore, FunctionKey


@pytest.fixture()
def fresh_cache(tmp_path, monkeypatch):
    monkeypatch.setenv("KERMAC_AMD_CACHE_DIR", str(tmp_path))
    mc.Singleton._instances.pop(mc.ModuleCache, None)
    yield tmp_path
    mc.Singleton._instances.pop(mc.ModuleCache, None)


def test_function_names_are_template_ids():
    name = mc.build_kernel_function_name(0, 1, 0, 2)
    assert name == "kmc::build_kernel<kmc::OP_DIFF,kmc::POW_ABS,kmc::LOAD_COL_VEC,kmc::LOAD_ROW_VEC>"
    d = kermac.kernel_descriptor_p_norm
    assert d._render_function_name(kermac.Majorness.COL_MAJOR, kermac.Majorness.ROW_MAJOR, kermac.Alignment.ALIGN_4,
                                   kermac.Alignment.ALIGN_1) == \
        "kmc::build_kernel<kmc::OP_DIFF,kmc::POW_POW,kmc::LOAD_COL_VEC,kmc::LOAD_ROW_SCALAR>"


def test_jit_compile_and_persist(fresh_cache):
    cache = kermac.ModuleCache()
    assert kermac.ModuleCache() is cache                          # singleton
    names = [mc.build_kernel_function_name(0, 3, 0, 0), mc.build_kernel_function_name(1, 2, 1, 3)]
    assert cache.compile_and_cache_functions(None, names)
    files = sorted(p.name for p in fresh_cache.iterdir())
    assert sum(n.startswith("fn-") for n in files) == 2           # one mapping per function
    assert sum(n.startswith("code-") for n in files) == 1         # one program, one code object
    assert "source_hash" in files
    for name in names:
        lowered, code_hash = cache._store.get_function_mapping(cache._key(name))
        assert lowered.startswith("_ZN3kmc12build_kernel")
        code = cache._store.get_code(code_hash)
        assert code[:4] == b"\x7fELF" and lowered.encode() in code
    # a second request compiles nothing: the code object file is untouched
    before = {p.name: p.stat().st_mtime_ns for p in fresh_cache.iterdir()}
    assert cache.compile_and_cache_functions(None, names)
    assert before == {p.name: p.stat().st_mtime_ns for p in fresh_cache.iterdir()}
    # and a new process-wide instance finds the entries on disk
    mc.Singleton._instances.pop(mc.ModuleCache, None)
    again = kermac.ModuleCache()
    assert again is not cache
    assert again._store.get_function_mapping(again._key(names[0])) is not None


def test_source_hash_change_clears_the_store(tmp_path):
    store = CodeObjectStore(tmp_path, "hash-one")
    key = FunctionKey("kermac_amd", "0.1.0", "7.0", "gfx950", "-O3", "kmc::f<1>")
    code_hash = store.put_code(b"\x7fELFfake")
    store.put_function_mapping(key, "_Zf", code_hash)
    assert store.get_function_mapping(key) == ("_Zf", code_hash)
    assert CodeObjectStore(tmp_path, "hash-one").get_function_mapping(key) == ("_Zf", code_hash)
    cleared = CodeObjectStore(tmp_path, "hash-two")                # headers changed
    assert cleared.get_function_mapping(key) is None and cleared.get_code(code_hash) is None
    assert (tmp_path / "source_hash").read_text() == "hash-two"


def test_damaged_code_object_is_dropped_not_returned(tmp_path):
    store = CodeObjectStore(tmp_path, "hash-one")
    key = FunctionKey("kermac_amd", "0.1.0", "7.0", "gfx950", "-O3", "kmc::f<1>")
    code_hash = store.put_code(b"\x7fELFfake-code-object")
    store.put_function_mapping(key, "_Zf1", code_hash)
    path = tmp_path / f"code-{code_hash}.hsaco"
    path.write_bytes(b"\x7fELFfake")                      # truncated behind the store's back
    assert store.get_code(code_hash) is None              # bytes no longer hash to the name
    assert not path.exists()
    assert store.get_function_mapping(key) is None        # so the function counts as not compiled


def test_key_covers_everything_the_binary_depends_on(tmp_path):
    store = CodeObjectStore(tmp_path, "h")
    base = dict(package_name="kermac_amd", package_version="0.1.0", toolchain_version="7.0", arch="gfx950",
                flags="-O3", function_name="kmc::f<1>")
    code_hash = store.put_code(b"x")
    store.put_function_mapping(FunctionKey(**base), "_Zf", code_hash)
    for field in base:
        other = dict(base, **{field: base[field] + "x"})
        assert store.get_function_mapping(FunctionKey(**other)) is None, field
    record = json.loads(next(tmp_path.glob("fn-*.json")).read_text())
    assert record["key"] == base


def test_compile_error_is_reported(fresh_cache):
    from kermac_amd import _backend
    with pytest.raises(_backend.BackendError) as info:
        _backend.jit_compile("__global__ void k() { this is not C++; }", "bad.hip", [], ["--offload-arch=gfx950"], [])
    assert info.value.status >= 2000 and "error" in str(info.value)


def test_pre_compile_descriptors_skips_aot_and_compiles_the_rest(fresh_cache):
    odd = kermac.KernelDescriptor(kermac.InnerOperator.DIFF, kermac.PowerType.SQRT, kermac.PowerType.NOOP,
                                  kermac.KernelType.NONE)
    kermac.pre_compile_descriptors(None, [kermac.kernel_descriptor_l1_norm, odd], try_to_align=False)
    mappings = list(fresh_cache.glob("fn-*.json"))
    assert len(mappings) == 4                                       # 2 x 2 unaligned layouts of `odd` only

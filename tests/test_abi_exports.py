"""The C-ABI library loads on a machine without a GPU and exports every symbol the public headers declare."""
import ctypes
import glob
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    names = []
    for header in sorted(glob.glob(os.path.join(ROOT, "include", "*.h"))):
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        for m in re.finditer(r"\b(thor(?:hip)?_[a-z0-9_]+)\s*\(", text):
            name = m.group(1)
            if name.endswith("_fn") or name.endswith("_t"):
                continue
            names.append(name)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    from thor_amd import _lib
    lib = _lib.load()
    declared = _declared_functions()
    assert len(declared) >= 30
    missing = [n for n in declared if not hasattr(lib, n)]
    assert not missing, f"declared in include/*.h but not exported: {missing}"


def test_prototype_table_covers_thorhip_header():
    from thor_amd import _lib
    declared = [n for n in _declared_functions() if n.startswith("thorhip_")]
    assert sorted(_lib.THORHIP_PROTOTYPES) == declared


def test_no_gpu_calls_fail_cleanly():
    from thor_amd import _lib
    lib = _lib.load()
    assert lib.thorhip_abi_version() == 1
    assert lib.thorhip_dtype_size(11) == 4 and lib.thorhip_dtype_size(24) == 2 and lib.thorhip_dtype_size(99) == -1
    n = ctypes.c_int(-1)
    assert lib.thorhip_device_count(ctypes.byref(n)) == 0 and n.value >= 0
    # argument validation happens before any device work
    assert lib.thorhip_convert(None, None, 11, 11, 4, None) != 0
    assert b"dtype" in lib.thorhip_last_error()
    assert lib.thorhip_convert(None, None, 11, 10, -1, None) != 0
    assert lib.thorhip_convert(None, None, 11, 10, 0, None) == 0


def test_runtime_compile_for_gfx950_without_a_device():
    """hipRTC cross-compiles on a CPU-only host, so the emitter's output can be syntax-checked here."""
    from thor_amd import _lib
    lib = _lib.load()
    src = b'extern "C" __global__ void k(const float* a, float* o, unsigned n) { unsigned i = blockIdx.x * blockDim.x + threadIdx.x; if (i < n) o[i] = a[i] * 2.0f; }'
    code, size = ctypes.c_void_p(), ctypes.c_size_t()
    log = ctypes.create_string_buffer(4096)
    rc = lib.thorhip_compile(src, b"probe.hip", b"gfx950", None, 0, ctypes.byref(code), ctypes.byref(size), log, 4096)
    assert rc == 0, lib.thorhip_last_error()
    assert size.value > 0
    lib.thorhip_code_free(code)
    bad = b'extern "C" __global__ void k() { this is not C++ }'
    rc = lib.thorhip_compile(bad, b"bad.hip", b"gfx950", None, 0, ctypes.byref(code), ctypes.byref(size), log, 4096)
    assert rc != 0 and b"error" in lib.thorhip_last_error()

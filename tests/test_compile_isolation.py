"""thorhip_compile with compile isolation: the compiler runs in a worker process, so a source that makes the compiler abort
(an internal compiler error ends in abort()) fails that one compilation with an error and leaves this process alive.  Needs no
GPU: the run-time compiler cross-compiles for gfx950."""
import ctypes

import pytest

from thor_amd import _lib

# With packed fp32 operations switched off (every kernel of this library is compiled that way), the compiler cannot select the
# <2 x float> operation its vectoriser builds from two fp32 -> fp16 conversions that feed packed fp16 arithmetic, and aborts with
# "Cannot select: v2f32 = bitcast".  (Generated kernels avoid the pattern by spelling the conversion as one instruction.)
ABORTS_THE_COMPILER = b"""
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
extern "C" __global__ void k(const h8* x, const h8* y, h8* o) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    h8 a = x[i], b = y[i], r;
#pragma unroll
    for (int k = 0; k < 8; ++k) r[k] = a[k] - (_Float16)__builtin_logf((float)b[k]);
    o[i] = r;
}
"""
GOOD = b'extern "C" __global__ void k(const float* a, float* o, unsigned n) { unsigned i = blockIdx.x * blockDim.x + threadIdx.x; if (i < n) o[i] = a[i] * 2.0f; }'


def compile_for_gfx950(lib, source, name):
    code, size = ctypes.c_void_p(), ctypes.c_size_t()
    log = ctypes.create_string_buffer(8192)
    rc = lib.thorhip_compile(source, name, b"gfx950", None, 0, ctypes.byref(code), ctypes.byref(size), log, 8192)
    error = lib.thorhip_last_error().decode(errors="replace") if rc != 0 else ""
    if rc == 0:
        lib.thorhip_code_free(code)
    return rc, size.value, error


@pytest.fixture()
def isolated():
    lib = _lib.load()
    before = lib.thorhip_set_compile_isolation(1)
    yield lib
    lib.thorhip_set_compile_isolation(before)


def test_a_compiler_abort_is_an_error_not_the_end_of_the_process(isolated):
    rc, size, error = compile_for_gfx950(isolated, ABORTS_THE_COMPILER, b"aborts.hip")
    assert rc != 0 and size == 0
    assert "signal" in error and "Cannot select" in error, error
    # the process and the library go on working
    rc, size, _ = compile_for_gfx950(isolated, GOOD, b"good.hip")
    assert rc == 0 and size > 0


def test_isolated_compiles_give_code_objects_and_logs(isolated):
    rc, size, _ = compile_for_gfx950(isolated, GOOD, b"good.hip")
    assert rc == 0 and size > 1000
    rc, _, error = compile_for_gfx950(isolated, b'extern "C" __global__ void k() { this is not C++ }', b"bad.hip")
    assert rc != 0 and "error" in error
    # the same code object as the in-process compiler produces
    lib = isolated
    lib.thorhip_set_compile_isolation(0)
    rc_in, size_in, _ = compile_for_gfx950(lib, GOOD, b"good.hip")
    lib.thorhip_set_compile_isolation(1)
    assert rc_in == 0 and size_in == size

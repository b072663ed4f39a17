"""thor_amd -- MI355X (gfx950) backend for Thor's Expression / reduction / TypeConverter hot path.

Python here is a thin mirror of the reference's `thor.physical` surface over the library's C ABI; the arithmetic lives
in libthor_amd.so (HIP kernels + the C++ Expression compiler).
"""
from .dtypes import DataType  # noqa: F401

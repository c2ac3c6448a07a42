"""MI355X-native GQA flash-attention path of the orin_llm engine.

The product is liborin_fa.so: hand-written gfx950 HIP kernels behind the C ABI of
include/orin_fa.h and a C++ shim with the reference's llm::cuda signatures.  This
package is the Python-side harness over that ABI (tests, benchmark); it holds no
compute of its own and has no CPU fallback.
"""
from . import kernels  # noqa: F401

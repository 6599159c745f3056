"""MI355X-native Gaussian-splat rasterizer hot path: host-side Python entry points.

`scenes` builds the seeded synthetic inputs; `lib` binds the C ABI of the HIP library
(csrc/libssr_hip.so, declared in include/ssr_backend.h); `host` binds the C++ host layer that
mirrors the reference's backend interface and engine call order.
"""
from . import scenes  # noqa: F401

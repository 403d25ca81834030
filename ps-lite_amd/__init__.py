"""pskv: the MI355X-native server-side key-value data path of a ps-lite style
parameter server. The product is libpskv.so (HIP for gfx950, C ABI in
include/pskv/capi.h) plus the C++ adapters in include/pskv; this package holds
the sources, the build recipe and a thin ctypes binding used by tests and the
benchmark."""
from . import build, capi, meta  # noqa: F401

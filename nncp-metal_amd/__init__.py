"""MI355X-native backend for NNCP's online-learning Transformer-XL step behind
the libnc C ABI.  The compute lives in csrc/libnc_hip.so (HIP, gfx950); this
package holds the ctypes binding and the host-side mirror of the reference's
model interface."""
from . import binding  # noqa: F401
from . import host  # noqa: F401,E402

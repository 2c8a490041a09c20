"""allpaka_amd -- MI355X (gfx950) implementation of allpaka's fused per-layer ops.

The product is `libapk_hip.so` (C ABI in include/apk_hip.h: hand-written HIP
kernels in an embedded gfx950 code object + a thin host runtime).  This Python
package is the host-side mirror of the reference's operator surface
(`allpaka_backend::ops`, `QuantMat::row_into`, `model::route_gated`, the
`gpu::*` decline convention) over that ABI; torch is used only to own device
memory.  There is no CPU fallback: without the built library every entry
raises.
"""
from .lib import ApkError, Declined, load, lib_path  # noqa: F401
from .backend import Backend, QuantMat, Gating, GgmlType  # noqa: F401

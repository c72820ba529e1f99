"""MI355X (gfx950) backend for gufo-npu's quantized matrix-vector decode path.

The product is the C-ABI library built from csrc/ (include/gufo_hip.h) and the C++
adapter in host/ that mirrors the reference's `qwen35::Projections`.  This Python
package only holds what drives them from tests and the bench: the ctypes binding
(capi), the seeded synthetic inputs (synth) and the build recipe (build).

The directory name carries a hyphen, so the package is loaded by path under the
module name `gufo_npu_amd` (see load_package in __graft_entry__.py).
"""

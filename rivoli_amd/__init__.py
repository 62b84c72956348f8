"""rivoli's fp8 MLA KV-cache hot path for MI355X (gfx950).

The product is the C-ABI library built from rivoli_amd/csrc (declared in include/*.h). This
package is the thin host-side mirror of the reference's launcher wall: `hip` holds one
`launch_*` per entry point (the names crates/backend/src/hip_attn.rs gives them) and
`pagepool` the host allocator that produces block tables and slot mappings.
"""
from . import hip, pagepool  # noqa: F401

__all__ = ["hip", "pagepool"]

"""pagedserve_amd: a single-GPU paged-KV inference engine for MI355X (gfx950)."""

__version__ = "0.1.0"

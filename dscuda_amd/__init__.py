"""MI355X-native attention hot path of dscuda: MLA forward / backward / decode
and causal flash-attention forward as hand-written gfx950 HIP kernels behind
the reference's C-ABI.  ``dscuda_amd.harness`` holds the ctypes caller that
mirrors the reference's ``benchmarks/`` harness; ``dscuda_amd.build`` compiles
the libraries."""

__all__ = ["build", "harness"]

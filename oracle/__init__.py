"""CPU restatement of the reference's arithmetic for the adapter-augmented SDXL UNet hot path.

TEST INFRASTRUCTURE ONLY.  This package is the checker for the HIP kernels: it is imported by
tests/, by `__graft_entry__.smoke()` and by the `cpu_baseline` leg of bench.py, and by nothing in
the product package.  Everything here is plain PyTorch on the CPU in fp32/fp64, written from the
reference's Python sources (each function cites the file:line it follows).
"""

"""CPU restatement of the reference's arithmetic for the adapter-augmented SDXL UNet hot path.

TEST INFRASTRUCTURE ONLY.  This package is the checker for the HIP kernels: it is imported by
tests/, by `__graft_entry__.smoke()` and by the `cpu_baseline` leg of bench.py, and by nothing in
the product package.  Everything here is plain PyTorch on the CPU in fp32/fp64, written from the
reference's Python sources (each function cites the file:line it follows).

What pins it (tests/test_oracle_*.py):
  ops.py        closed forms, library routines (F.scaled_dot_product_attention, F.group_norm, F.layer_norm,
                F.gelu), fp64 brute force, the invariants of the reference's LoRA test-suite
  blocks.py     15 seeded known-answer slices of the reference's unit tests
  euler.py      3 full-loop known answers of the reference's scheduler tests
  unet_sdxl.py  structure: the 722 LoRA-able linears of the reference's key-match fixture, skip shapes
  controlnet.py structure: zero output when fresh, from_unet identity, residual shapes

Parity unpinned (no runnable reference test or fixture covers it offline):
  * end-to-end numbers of unet_sdxl.UNet2DConditionModel and controlnet.ControlNetModel on real
    checkpoints (the reference's goldens for them need hub weights); their blocks are pinned, their
    wiring is pinned structurally only;
  * the dtype-cast order inside peft's Linear.forward (third-party, absent); immaterial inside the
    bf16 tolerance of the tests.
"""

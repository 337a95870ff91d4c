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
  unet_sdxl.py  the forward, numerically: outputs of the reference's own UNet2DConditionModel on a tiny
                SDXL-topology configuration, with and without the 9 + 1 ControlNet residuals, <= 1e-4
                (tests/golden/unet_tiny_reference.safetensors, written by tests/golden/make_unet_tiny_fixture.py from
                the reference's modules; weights and inputs are functions of tensor names, tests/helpers.py);
                structure: the 722 LoRA-able linears of the reference's key-match fixture, skip shapes
  controlnet.py the forward, numerically: the reference's ControlNetModel (from_unet, non-zero zero-convs), same
                fixture, <= 1e-4 relative; zero output when fresh, from_unet identity, residual shapes

Parity unpinned (no runnable reference test or fixture covers it offline):
  * the dtype-cast order inside peft's Linear.forward (third-party, absent from the image); immaterial inside the
    bf16 tolerance of the tests.  The LoRA arithmetic itself is pinned by the closed form of the reference's in-repo
    LoRALinearLayer / LoRACompatibleLinear, fp64 brute force and the merge identity (tests/test_oracle_ops.py).
The full-size SDXL models are the same code as the tiny configuration with other widths and depths; no reference
output at full size exists offline (its goldens need hub checkpoints), which the fixture above does not change.
"""

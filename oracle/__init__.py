"""CPU oracle for the fused quantised-LoRA path.  TEST INFRASTRUCTURE ONLY.

Nothing under this package is part of the product: it may be imported by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py`` -- as the checker,
never as the thing that is measured or shipped.  The product path (``fms-acceleration_amd/``)
never imports it and fails loudly when its HIP library is missing.

Every function restates a piece of the reference and cites the file:line it follows
(paths relative to the reference checkout):

  FOAK = plugins/fused-ops-and-kernels/src/fms_acceleration_foak
  UL   = FOAK/fused_ops/unsloth_lora
  GQ   = plugins/accelerated-peft/src/fms_acceleration_peft/gptqmodel

How each function is pinned (the reference holds no numeric fixtures for this path, and its own
parity tests need hub checkpoints, a CUDA GPU, peft, bitsandbytes and auto_gptq, none of which is
available offline -- so nothing from the reference was imported or executed):

  gptq.pack_rows / pack_cols / unpack_*   closed form of pack(); brute force bit-by-bit on tiny
                                          shapes; pack o unpack = identity          (test_oracle_gptq)
  gptq.dequant                            exact integer/fp64 arithmetic; v1/v2 zero-point identity
                                          (zero_offset=1 == qzeros + 0x11111111); act-order joint
                                          permutation invariance; per-element scalar loop
  gptq.rtn_quantize                       closed form; invariants |W - deq| <= scale/2 inside the
                                          clamp range, zero in [0, 15], symmetric special case
  lora.*  (forward / backward)            torch.autograd of the unfused graph vs the hand-derived
                                          formulas in fp64; finite differences; special cases B=0,
                                          A=0, linearity in s, adapters disabled
  swiglu.*                                torch.nn.functional.silu and its autograd
  nf4.dequant / quantize                  closed form + round trip.  The 16-entry NF4 table and the
                                          nibble order are bitsandbytes facts (module
                                          `bitsandbytes`, >=0.45.1 in
                                          plugins/accelerated-peft/requirements.txt:10), absent from
                                          the reference tree: PARITY UNPINNED beyond the published
                                          table; the 256-entry double-quant codebook is an input.
"""

"""CPU oracle of the FlagRot KV-cache hot path (numpy only).

TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
import this package, and only as the checker / the timed CPU baseline.  The product path is the HIP library behind
the C ABI in include/; it never calls into this package and fails loudly when its shared library is missing.

Modules
  quant    fwht, symmetric / asymmetric group quantisers, scale words, static writer, key-only 2x2 selecting
           encoder, whole-head Hadamard            (follows kernels/ref.py, kernels/codebook_ref.py,
                                                    blockflag/formats.py, blockflag/hadamard.py of the reference)
  pages    byte-exact page packers and independent parsers of the 144 P (INT4) and 80 P (INT2) chunk layouts
                                                   (follows kernels/csrc/attn_decode_v2.cuh:14-46 of the reference)
  attend   dequantise-then-attend reference, split merge
                                                   (follows integrations/vllm_flagrot/tests/test_kernels.py:37-56)
  kivi     KIVI-style INT2 quantisers, page layout, dequantiser, attention reference
                                                   (follows integrations/vllm_flagrot/csrc/kivi.cu:1-35,94-125 and
                                                    vllm_flagrot/kivi.py:184-308)
  mq       causal multi-query prefill reference over dequantised pages
                                                   (follows integrations/vllm_flagrot/scripts/bench_mq_prefill.py:82-95)

Parity status of every function is stated in its module header ("pinned by ..." or "parity unpinned").
"""

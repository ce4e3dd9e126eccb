"""CPU oracle of the paged-KV attention path: TEST INFRASTRUCTURE ONLY.

Importable from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg; the product package (llama_lite_npu_amd) must never import it.

  c_oracle  -- ctypes wrapper over litekv_oracle.c (plain C, OpenMP)
  cpu_ref   -- PyTorch-CPU restatement of the reference's torch functions
"""

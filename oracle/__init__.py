"""CPU restatement of the reference's flash-attention arithmetic.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: it is the checker used by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``.  The product path is the HIP
library and fails loudly when that library is missing.

Modules
-------
philox     Philox-4x32-10 and the dropout keep-mask closed form
           (reference: modules/flash/kernel/dropout.py:16-71).
intervals  parse_window / calculate_intervals
           (reference: modules/flash/kernel/masked_load_store.py:25-210).
fa_ref     attention forward/backward in fp32/fp64 with explicit masks, LSE,
           delta (reference kernels fwd_kernel.py, bwd_kernel_*.py; the
           reference's own test oracle _common_test.py:61-79).

Pinning status (what fixes each function independently of this file):
  philox4x32_10      Random123 known-answer vectors (three), tests/test_oracle_philox.py
  dropout word order Triton-interpreter probe values recorded for seed 0x1234
                     (tests/golden/philox_seed1234.json)
  idropout_p         probe value -1717986944 for p=0.1 and closed form for 0.5/0.2
  visible mask       brute force against torch tril/triu special cases
  intervals          brute force: union of block ranges == blocks with a visible
                     element; full blocks hold no masked element
  fa_ref fwd/bwd     torch.ops.aten._scaled_dot_product_attention_math + autograd
                     (library routine), LSE known answer 2.79018449783325195
Whole-tensor golden masks from the reference kernel itself do not exist in the
reference tree, so the dropout mask has no reference-held fixture: it is pinned
by derivation + probe values + known-answer vectors only.
"""

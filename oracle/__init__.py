"""CPU oracle for the GEMM / mask-based implicit-GEMM sparse-convolution path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is used by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU baseline.

Every function restates, in numpy (plus a few lines of C for the float
operations whose rounding must be fixed), what the reference computes; the
reference file:line each one follows is cited in its docstring.

Pinning status (how each part is anchored other than by re-typing itself):

* dense / ShuffleAC / ShuffleAB GEMM      - textbook ``A @ B`` identities, tests/test_oracle_gemm.py
* sparse fwd / dgrad / wgrad              - dense ``conv3d`` (torch CPU) + autograd on small grids
* tile mask / mask_output / reverse mask  - integer closed forms + brute force
* int8 epilogue                           - exhaustive check of round-half-even + saturation
* bf16 rounding                           - torch.bfloat16 conversion on random + tie values
* descriptor names / workspace / mnk      - the reference's own headers compiled into oracle/_ref
* stand-alone gather / scatter-add         - permutation + inverse, identity index, one-hot matrix
  product, index counts, f16 tie rounding; tests/test_oracle_gather.py
* pair tables (SubM and strided)          - PARITY UNPINNED against spconv (not part of the
  reference tree); pinned only against a brute-force dictionary search, and the
  row order of strided outputs / argsort tie-breaking are this build's conventions.
"""

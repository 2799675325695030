"""Process-wide numerics switch, same meaning as the reference's
models/global_config.py:1-6.

  0, 1 : attention softmax/aggregation by the per-crystal torch loop
  >= 1 : mean pooling by the irregular-mean kernel
  >= 2 : fused dot-product attention kernel
  >= 3, >= 4 : accepted; the HIP kernels have a single (blocked/tree)
         summation order, so these select nothing further.
"""
REPRODUCIBLITY_STATE: int = 3

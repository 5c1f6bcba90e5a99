"""Constants of the reference's constants.py:1-2, kept under the same names.

``dimension_numbers`` is the A.B^T contraction spec the reference hands to ``lax.dot_general``;
``MIN_BLOCK_SIZE`` is the reference's minimum tile edge (a TPU lane width there; here the
granularity callers' block sizes are validated against).  ``DEFAULT_MASK_VALUE`` is the additive
mask value of flex_attention_kernel.py:288; the HIP kernels use -inf with an all-masked-row guard,
which gives the same result for every row that keeps at least one key.
"""
import numpy as np

dimension_numbers = (((1,), (1,)), ((), ()))
MIN_BLOCK_SIZE = 128
DEFAULT_MASK_VALUE = -0.7 * float(np.finfo(np.float32).max)

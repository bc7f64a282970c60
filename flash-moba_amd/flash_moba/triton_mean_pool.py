"""Import-compatibility module: the reference exposes ``flash_topk_mean_pool`` from
``flash_moba.triton_mean_pool`` (flash_moba/triton_mean_pool.py:112).  Here the kernel
behind it is a HIP kernel (csrc/mean_pool.hip); no Triton is involved."""
from flash_moba.mean_pool import flash_topk_mean_pool  # noqa: F401

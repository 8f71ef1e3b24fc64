"""``ninetoothed.utils.calculate_default_configs`` (src/ninetoothed/utils.py:4-12).

The reference derives the default ``num_warps`` / ``num_stages`` of its Triton configurations
from the device's shared memory (8 warps, one stage per 32 KiB).  ``make`` accepts both arguments
and ignores them -- the kernels of ``libnt_hip.so`` have their wave counts and LDS rings built
in -- so the function only answers the same question for this part: a CU of gfx950 has 160 KiB of
LDS, which the largest GEMM instance uses as a ring of five 32 KiB stages, with eight waves per
workgroup."""

LDS_BYTES_PER_CU = 160 * 1024


def calculate_default_configs():
    """``(num_warps, num_stages)`` by the reference's rule on this part's LDS size."""
    return 8, LDS_BYTES_PER_CU // 2**15

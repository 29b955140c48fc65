"""MI355X (gfx950) Shfl-BW sparse inference: row-permuted vector-wise block-sparse fp16 SpMM and
implicit-GEMM sparse Conv2D.  The product is the HIP library behind the C ABI of include/shflbw.h
(csrc/); this package only holds the ctypes binding and a host-side mirror of the reference's
operator interface used by the tests and the benchmark."""
from . import capi
from .host import (BlockwiseSpFilter, BlockwiseSpMatrix, SpconvBlockwiseOp, SpmmBlockwiseOp, device_info,
                   random_mask, spconv_variant_name, spconv_variants, spmm_variants)

__all__ = ["capi", "BlockwiseSpMatrix", "BlockwiseSpFilter", "SpmmBlockwiseOp", "SpconvBlockwiseOp", "random_mask",
           "spmm_variants", "spconv_variants", "spconv_variant_name", "device_info"]

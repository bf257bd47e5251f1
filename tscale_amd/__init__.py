"""tscale_amd: MI355X (gfx950) implementation of TScale's quantized attention path.

The product is the HIP library `tscale_amd/lib/libtsattn.so` behind the C ABI of `include/tsattn.h`.
`tscale_amd.attention` is the Python host-side mirror of the reference's attention call sites, used
by the parity tests and the benchmark; torch only provides device memory and streams.
"""
from . import capi  # noqa: F401
from .attention import AttentionContext, KVCache  # noqa: F401

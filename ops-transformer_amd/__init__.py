"""MI355X-native quantized MoE expert-FFN path behind the reference's aclnn C entry points.

The product is ``lib/libcust_opapi.so`` (HIP kernels for gfx950 + the two-phase aclnn C-ABI, built by ``build.py``).
This package is the Python host layer over it: ``aclnn`` binds the C symbols with ctypes and exposes one function per
operator with the reference operator's argument names; ``moe_ffn`` chains the four operators into the expert FFN;
``synth`` generates the seeded synthetic workloads the benchmark and the tests run on.

The directory name contains a hyphen, so it is loaded by path (``__graft_entry__.load_package()``) and registered as
``ops_transformer_amd``.  torch is used for device memory and streams only.
"""
from . import aclnn, moe_ffn, synth  # noqa: F401
from .aclnn import (AclnnError, grouped_matmul_swiglu_quant, grouped_matmul_v4, library_path, moe_finalize_routing_v2,  # noqa: F401
                    moe_init_routing_v2)
from .moe_ffn import MoeFfnW8A8  # noqa: F401

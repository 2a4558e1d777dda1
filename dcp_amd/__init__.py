"""MI355X-native execution path for DCP's per-device blockwise attention.

``dcp_amd.ops`` mirrors ``dcp.ops`` (fused block copy / merge / sum),
``dcp_amd.flash_attn_interface`` mirrors the paged range-masked attention of
the reference's flash-attention fork, and ``dcp_amd.runtime.flash_attention``
mirrors the executor that drives them from an ``ExecutionPlan``.  All compute
runs in hand-written gfx950 HIP kernels behind the C ABI of ``libdcp_hip.so``.
"""

__version__ = "0.1.0"

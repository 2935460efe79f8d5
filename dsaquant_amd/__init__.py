"""dsaquant_amd -- the W4A4 linear hot path of DSAQuant, native to AMD MI355X.

Sub-packages mirror the reference's module paths for this path:

    dsaquant_amd.kernels.vdm_w4a4              <-> vdm_infer/kernels/vdm_w4a4.py
    dsaquant_amd.quantization.quant_linear     <-> vdm_infer/quantization/quant_linear.py
    dsaquant_amd.checkpoints.packed_checkpoint <-> vdm_infer/checkpoints/packed_checkpoint.py
    dsaquant_amd.fused_qkv                     <-> _get_qkv_projections in
                                                   vdm_infer/models/wan_vdm/modules/attention.py

The arithmetic lives in ``libvdmq.so`` (HIP, gfx950), reached through the C ABI
declared in ``include/vdmq.h``.  There is no CPU or PyTorch fallback for the
kernel path: without the library the kernel functions raise.
"""

__all__ = ["kernels", "quantization", "checkpoints", "fused_qkv"]

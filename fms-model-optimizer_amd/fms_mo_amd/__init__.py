"""MI355X-native (gfx950) implementation of fms-model-optimizer's quantized-linear inference path.

Layout mirrors the reference package for the modules on that path:
  fms_mo_amd.modules.linear            QLinear, QLinearINT8Deploy, LinearFPxAcc, QLinearINT8Train
  fms_mo_amd.modules.fp8_linear        FP8Linear
  fms_mo_amd.quant.quantizers          the quantizer subset those modules need
  fms_mo_amd.custom_ext_kernels.utils  torch.ops.fms_mo.* registration, lowering helpers
  fms_mo_amd.custom_ext_kernels.hip_kernels  matmul_chunk_truncate (the tl_matmul_chunk_truncate API)
  fms_mo_amd.modules.bmm               QBmmINT8Deploy (attention matmuls)
  fms_mo_amd.aiu_addons.i8i8           torch.ops.fms_mo.i8i8_aiu, W8A8LinearAIU
  fms_mo_amd.aiu_addons.fp8            torch.ops.spyre.scaled_bmm
  fms_mo_amd.utils.aiu_utils           AIU-style int8 checkpoint writer / reader
  fms_mo_amd.quant.ptq                 SmoothQuant activation statistics
  fms_mo_amd.kernels / fms_mo_amd._lib tensor-level and ctypes bindings of libfmsmo_hip.so
"""
__version__ = "0.1.0"

"""Drop-in name: ``import feather`` resolves to the MI355X implementation in
``feather_amd`` (same module paths as the reference package)."""
from feather_amd import *  # noqa: F401,F403
from feather_amd import (__version__, dot, flash_attention_fp8_acc_fp32_gpu,  # noqa: F401
                         flash_attention_fp8_e4m3_acc_fp32_gpu, flash_attention_fp8_e5m2_acc_fp32_gpu, gemv,
                         pack_fp8_tensor, pack_fp16_tensor, paged_attention_fp8_acc_fp32_gpu, unpack_fp8_tensor,
                         unpack_fp16_tensor)

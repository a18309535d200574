"""MI355X-native causal flash attention behind Sentinel's CudaFlashAttention interface."""
from .flash_attention import (  # noqa: F401
    HipAmp,
    HipFlashAttention,
    HipOps,
    collect_kernel_timings,
    decode_attention,
    flash_attention_backward,
    flash_attention_forward,
    library_path,
    load_library,
    set_kernel_timing,
)

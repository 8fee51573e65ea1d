from .ops import (  # noqa: F401
    QuantState,
    get_device_count,
    get_device_info,
    get_load_error,
    is_available,
    sdpa_decode,
    sdpa_prefill,
    sdpa_prefill_fused,
    sdpa_prefill_fused_v2,
)
from .sdpa import HipMultiHeadSelfAttention, HipSDPA, can_do_hip_sdpa, get_hip_sdpa  # noqa: F401

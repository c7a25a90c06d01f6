"""MI355X-native Mamba-2 SSD chunk-scan forward and streaming step (hand-written gfx950 HIP
kernels behind the C ABI in include/ssd_hip.h)."""
from .ssd import (  # noqa: F401
    PreparedChunkScan,
    SsdError,
    chunk_cumsum,
    chunk_scan_stage,
    chunk_state,
    chunk_state_passing,
    load_library,
    ssd_chunk_scan,
    ssd_chunk_scan_backward,
    ssd_chunk_scan_onepass,
    ssd_step,
    ssd_steps,
    state_passing,
    workspace_bytes,
)
from .stream_state import SsdStreamState  # noqa: F401
from .block import (GraphedBlockStep, Mamba2Block, Mamba2StreamState, block_post, block_post_bwd, block_post_proj, block_pre,  # noqa: F401
                    block_pre_bwd, block_proj, block_step)

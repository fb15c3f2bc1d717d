"""MI355X-native Stream-K GEMM: Python host layer over libstreamk.so."""
from ._lib import LIB_PATH, StreamKError, kernel_name, lib, strerror  # noqa: F401
from .ops import (StreamKKernel, bench_ms, dequant_q4, graph_ms, pack_q4, quantize_q4, reset_workspaces,  # noqa: F401
                  streamk_bf16, streamk_fp8, streamk_fp16, streamk_fp32, streamk_int8, streamk_q4, tile_q4, timing_stream, tl_matmul_streamk, unpack_q4,
                  untile_q4, workspace_status)
from .autotune import autotune, candidate_configs  # noqa: F401
from .linear import StreamKLinear  # noqa: F401
from .plan import cta_range, make_config, make_plan, num_cus, tile_coords, tuned_config  # noqa: F401

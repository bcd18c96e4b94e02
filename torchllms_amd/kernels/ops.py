"""The kernels as functions of ``torch`` tensors: one name space over the modules that hold them.

Every function checks on the host that shapes, dtypes and devices are what the kernel and its grid
assume, launches on torch's current HIP stream and raises ``KernelError`` when a launcher refuses.
Tensors must live on the GPU: there is no CPU path.  Only what parts and callers use is named here;
a module's own helpers and tables stay in the module.

``base``             dtype codes, argument checks, ``Unfinished`` results (``SplitSums``)
``elementwise_ops``  embedding, RMS norm, rotary + cache write, gate, bias
``products``         matrix products and the measurement that picks their kernel
``attention_ops``    plain, decode and prefill attention with their launch plans
``sequence_ops``     layer norm with a scaled sum, gated activations, unit-norm rotation with the cache
                     write, short convolutions, selective scan, gated delta rule, matrix memory
``head_ops``         branches normed into a 32-bit stream, heads prepared before the scores (weighted norm, partial
                     rotation, query factor, mixed values), gates, packing for attention through a latent, logit cap
``routed_ops``       router (softmax scores, corrected choice), experts over the rows that chose them, bias with the
                     exact gelu, the norm behind a branch together with the norm before the next
``stream_ops``       several residual streams with their weighted reads and writes, the norm without statistics,
                     the join of differential attention's two maps
``sampling_ops``     the sampling kernel
"""

from .base import (  # noqa: F401
    BF16,
    F32,
    KernelError,
    SplitSums,
    Unfinished,
    check,
    core,
    device_facts,
    dtype_code,
    resolved,
    variant,
)
from .elementwise_ops import (  # noqa: F401
    rmsnorm_max_hidden,
    add_bias_,
    embed,
    rmsnorm,
    rope_kv_write,
    rope_table,
    silu_mul,
)
from .products import (  # noqa: F401
    LINEAR_USES,
    ROW_BUCKETS,
    STREAM_MAX_ELEMENTS,
    STREAM_MAX_ROWS,
    STREAM_WAVE_CHOICES,
    WIDE_CHOICES,
    WIDE_MAX_ROWS,
    clear_kernel_table,
    kernel_table,
    load_kernel_table,
    save_kernel_table,
    gemm_f32,
    gemm_stream,
    gemm_stream_glu,
    gemm_stream_qkv,
    gemm_stream_residual,
    NORMED_ROWS_MAX_WIDTH,
    NormedRows,
    PendingProduct,
    gemm_wide,
    gemm_wide_glu,
    gemm_wide_qkv,
    linear,
    linear_choice,
    linear_glu,
    linear_to_sum,
    qkv_rope_store,
    stream_supported,
    tune_linear,
    wide_fits,
    wide_supported,
)
from .attention_ops import (  # noqa: F401
    ATTENTION_MAX_HEAD_DIM,
    ATTENTION_MAX_KEY_DIM,
    DECODE_HEAD_DIMS,
    PREFILL_HEAD_DIMS,
    PREFILL_SPLIT_ALWAYS,
    PREFILL_SPLIT_BLOCKS,
    PREFILL_SPLIT_KEYS,
    attention_decode,
    attention_generic,
    attention_generic_split,
    attention_prefill,
    decode_attention_supported,
    plan_decode_splits,
    prefill_attention_supported,
    prefill_key_groups,
    prefill_queries_per_tile,
    prefill_tile_count,
    prefill_tiles,
)
from .sequence_ops import (  # noqa: F401
    SCAN_SEGMENTS_FROM,
    ScaledSum,
    ScanSegments,
    causal_conv,
    embed_scaled,
    gated_delta,
    gated_linear,
    gelu_mul,
    layernorm,
    matrix_memory,
    matrix_memory_state_size,
    rope_norm_kv_write,
    selective_scan,
    state_region,
)
from .head_ops import (  # noqa: F401
    HEAD_PREPARE_MAX_DIM,
    branch_norm_add,
    head_prepare,
    pack_heads,
    rmsnorm_columns,
    sigmoid_gate_,
    softcap_,
    unpack_heads_gate,
)
from .routed_ops import (  # noqa: F401
    ROUTER_MAX_OUTPUTS,
    bias_gelu_,
    expert_combine,
    expert_down_rows,
    expert_gather,
    expert_glu_rows,
    expert_pair_products,
    PAIR_PRODUCTS_MOST,
    post_norm_add_norm,
    router_topk,
    weighted_pair,
)
from .stream_ops import (  # noqa: F401
    MAX_STREAMS,
    maps_join,
    streams_open,
    streams_update,
)
from .sampling_ops import (  # noqa: F401
    philox_uniform,
    sample,
    sample_chunks,
)

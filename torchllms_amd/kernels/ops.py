"""The kernels as functions of ``torch`` tensors: one name space over the modules that hold them.

Every function checks on the host that shapes, dtypes and devices are what the kernel and its grid
assume, launches on torch's current HIP stream and raises ``KernelError`` when a launcher refuses.
Tensors must live on the GPU: there is no CPU path.  Only what parts and callers use is named here;
a module's own helpers and tables stay in the module.

``base``             dtype codes, argument checks, ``Unfinished`` results (``SplitSums``)
``elementwise_ops``  embedding, RMS norm, rotary + cache write, gate, bias
``products``         matrix products and the measurement that picks their kernel
``attention_ops``    plain, decode and prefill attention with their launch plans
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
from .sampling_ops import (  # noqa: F401
    philox_uniform,
    sample,
    sample_chunks,
)

"""The kernels as functions of ``torch`` tensors: one name space over the modules that hold them.

Every function checks on the host that shapes, dtypes and devices are what the kernel and its grid
assume, launches on torch's current HIP stream and raises ``KernelError`` when a launcher refuses.
Tensors must live on the GPU: there is no CPU path.

``base``             dtype codes, argument checks, ``SplitSums``
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
    _DTYPE_CODE,
    _gpu,
    _i32,
    _ptr,
    _stream,
    check,
    core,
    dtype_code,
    resolved,
    variant,
)
from .elementwise_ops import (  # noqa: F401
    _rmsnorm_split,
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
    _LINEAR_CHOICE,
    _TAIL_KERNEL_US,
    _TUNE_FLUSH_BYTES,
    _fuses_tail,
    _qkv_shapes,
    _row_bucket,
    _run_choice,
    _run_glu,
    _wide_shapes,
    gemm_f32,
    gemm_stream,
    gemm_stream_glu,
    gemm_stream_qkv,
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
    DECODE_HEAD_DIMS,
    PREFILL_HEAD_DIMS,
    PREFILL_RESIDENT_BLOCKS,
    PREFILL_SPLIT_BLOCKS,
    _DECODE_BLOCK_KEYS,
    _DECODE_MIN_SPLIT,
    _DECODE_SIGNATURES,
    _DECODE_UNEVEN_SPLIT,
    _F,
    _I,
    _P,
    _PREFILL_SIGNATURES,
    attention_decode,
    attention_generic,
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

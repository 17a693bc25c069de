"""MI355X (gfx950) backend for effect-torch's quantized-GGUF matmul path.

Import name: this directory is called ``effect-torch_amd``; load it with
``importlib`` (``tests/conftest.py`` and ``bench.py`` register it as
``effect_torch_amd``).
"""
from .quantized import (  # noqa: F401
    ActivationMode,
    CancellationFlag,
    Cancelled,
    EmbeddingRequirements,
    GgmlQuant,
    QuantizedError,
    QuantizedRequirements,
    LinearGroup,
    RawLinear,
    STATIC_WORKSPACE_BYTES,
    MFMA_OPERATIONS,
    CONTRACTION_PROBES,
    calibration_contraction,
    calibration_copy,
    calibration_mfma,
    calibration_read,
    calibration_read_variant,
    READ_VARIANTS,
    dequantize_rows,
    embedding_into,
    embedding_requirements,
    embedding_status_check,
    handover_timeouts,
    is_available,
    linear_into,
    linear_requirements,
    quantize_activations,
    quantized_linear,
    set_handover_spin_limit,
)
from .kv_cache import (  # noqa: F401
    KvLayer,
    kv_attention_into,
    kv_attention_kernel,
    kv_attention_projected_into,
    kv_attention_status_check,
    kv_attention_workspace,
    kv_attention_workspace_bytes,
    kv_commit,
)
from .decode_ops import (  # noqa: F401
    RotaryLayout,
    add_into,
    gather_rows_into,
    gather_rows_status_check,
    greedy_status_check,
    greedy_tokens,
    greedy_workspace_bytes,
    rms_norm_into,
    rotary_into,
    rotary_pair_into,
    silu_mul_into,
)
from .decode_step import LlamaDecoder, LlamaShape, algorithmic_bytes_per_step  # noqa: F401
from .gguf import (  # noqa: F401
    GgufFile,
    GgufMetadataValue,
    GgufParseError,
    GgufTensorDescriptor,
)

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
    RawLinear,
    calibration_copy,
    calibration_read,
    dequantize_rows,
    embedding_into,
    embedding_requirements,
    embedding_status_check,
    is_available,
    linear_into,
    linear_requirements,
    quantize_activations,
    quantized_linear,
)

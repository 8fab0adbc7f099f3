"""MI355X-native quantized projection operators (GGUF Q8_0 / Q4_K / Q6_K) behind a C ABI."""
from .qproj import (ACT_F32, ACT_GGML, ACT_Q8X32, TYPE_Q4_K, TYPE_Q6_K, TYPE_Q8_0, Context, QprojError,
                    Weight, load_library, row_bytes)

__all__ = ["ACT_F32", "ACT_GGML", "ACT_Q8X32", "TYPE_Q4_K", "TYPE_Q6_K", "TYPE_Q8_0", "Context",
           "QprojError", "Weight", "load_library", "row_bytes"]

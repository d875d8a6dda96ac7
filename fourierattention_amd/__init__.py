"""MI355X-native Fourier KV-cache hot path: cache object, decode attention and spectral
compression behind the reference's Python interface, computed by hand-written HIP kernels
(``libfourier_attn_hip.so``, C ABI in ``include/fourier_attn_hip.h``)."""
from .cache import Cache, DynamicCache, StaticCache, ExtraConfig, CacheParts  # noqa: F401
from .ops import (MultiDimHiPPO2, fourier_attn, mat_avg_std_triton, mat_fourier_avg_std_triton,  # noqa: F401
                  mat_fourier_inv, mat_fourier_triton, triton_fourier_attn)
from .attention import LlamaSdpaAttention, fourier_attention  # noqa: F401
from . import masks  # noqa: F401

__all__ = ["Cache", "DynamicCache", "StaticCache", "ExtraConfig", "CacheParts", "MultiDimHiPPO2", "fourier_attn", "triton_fourier_attn",
           "mat_fourier_triton", "mat_avg_std_triton", "mat_fourier_avg_std_triton", "mat_fourier_inv",
           "LlamaSdpaAttention", "fourier_attention", "masks"]

"""fastnn_amd: MI355X-native (gfx950) implementation of fastnn's weight-quantised MatMul
hot path behind a C ABI (libfastnn_hip.so), with a thin ctypes host layer."""
from .lib import (  # noqa: F401
    ACT_GELU, ACT_NONE, ACT_RELU, ACT_SILU, DT_F4, DT_F8, DT_F8R, DT_I4, DT_I4CB, DT_I8, DT_U4, DT_U8,
    FLAG_ACT_F16_SINGLE, FLAG_DEVICE_PTRS, FLAG_FORCE_GENERIC, FLAG_I4CB_AS_WRITTEN, FLAG_PREFER_FMA,
    FnnError, HipContext, PackedWeight, load_library, quantize_weights, quantize_weights_kn,
)
from .aot import AotExecutor, weight_dtype_of  # noqa: F401,E402

"""native-hip: MI355X (gfx950) tier for OxiBonsai's Q1_0_g128 / TQ2_0_g128 hot path.

The compute lives in ``lib/liboxb_hip.so`` (hand-written HIP behind a C ABI,
``include/oxb_hip.h``); this package is the host-side mirror of the reference's
backend interface used by the tests and the benchmark."""
from .backend import GpuError, GpuWeightHandle, NativeHipBackend, repack, unpack  # noqa: F401
from .synth import Q1, TQ2  # noqa: F401

"""MI355X-native paged / quantized KV-cache attention ops with AReno's op signatures.

Only the hot path lives here: ``areno_amd.accel`` (the ops the reference's
``areno.accel.attention`` exports, backed by hand-written HIP kernels for gfx950) and
``areno_amd.engine`` (the inference attention backend that calls them).
"""

__version__ = "0.1.0"

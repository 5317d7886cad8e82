"""Engine-side glue for the MI355X attention path: the metadata carrier, the paged (optionally quantized) KV-cache
allocation, the device-resident page bookkeeping and the inference attention backend module the model layers call.
Mirrors the shapes of areno/engine/runtime/metadata.py, areno/models/qwen3/model.py:309-333,
areno/engine/data/rollout_state.py (page lists) and areno/engine/layers/attention_backend/infer.py in the
reference."""

from areno_amd.engine.block_tables import DeviceBlockTables
from areno_amd.engine.attention_backend import HipInferBackend, build_infer_attention_backend
from areno_amd.engine.kv_cache import KVCacheLayer, allocate_kv_caches, kv_cache_bytes_per_token
from areno_amd.engine.metadata import InferMeta

__all__ = [
    "DeviceBlockTables",
    "HipInferBackend",
    "InferMeta",
    "KVCacheLayer",
    "allocate_kv_caches",
    "build_infer_attention_backend",
    "kv_cache_bytes_per_token",
]

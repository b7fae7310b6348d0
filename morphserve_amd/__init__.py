"""MI355X-native paged-KV hot path behind the SwiftLLM/MorphServe operator surface.

Drop-in names (reference file each mirrors):

* ``worker.kernels.kvcache_mgmt.store_kvcache``      MorphServe/worker/kernels/kvcache_mgmt.py
* ``worker.kernels.paged_attn.paged_attention``      MorphServe/worker/kernels/paged_attn.py
* ``worker.kernels.prefill_attn.prefill_attention``  MorphServe/worker/kernels/prefill_attn.py
* ``worker.kernels.rotary_emb.*``                    MorphServe/worker/kernels/rotary_emb.py (+ fused append)
* ``worker.kernels.block_mgmt.*``                    MorphServe/worker/kernels/block_mgmt.py
* ``worker.block_manager.BlockManager``              MorphServe/worker/block_manager.py
* ``worker.infer_state.LlamaInferState``             MorphServe/worker/infer_state.py
* ``model_config.LlamaModelConfig``                  MorphServe/model_config.py (attention geometry, ``get_kvslot_size``)
* ``swiftllm_c``                                     csrc/src/entrypoints.cpp (KV entries only)
* ``elastic_pool.ElasticKVPool``                     pool expand / shrink with live-block migration
* ``kv_placement.allocate_kv_caches``                MorphServe/worker/model.py:187-190 (the K and V pool allocation)
* ``vmm_pool.VmmKVPool``, ``vmm_pool.LayerArena``      the same pool as ONE tensor over HIP virtual memory; a layer's
                                                     memory moving into it and back (csrc/src/memory_manager.cpp:69-176)
* ``worker.layers.attention_section``                MorphServe/worker/layers/transformer_layer.py:93-191 (rotary .. decode attention)
* ``worker.swap.KVSwapper``                          MorphServe/worker/model.py:468-534 (sequence eviction)
* ``server.Scheduler``                               MorphServe/server/scheduler.py

All compute goes through ``libmorphkv.so`` (hand-written HIP for gfx950) via
ctypes; nothing here falls back to eager PyTorch.
"""
from . import _capi  # noqa: F401
from .model_config import LlamaModelConfig  # noqa: F401
from .worker.infer_state import (LlamaInferState, StepStateBuilder, build_infer_state,  # noqa: F401
                                 select_seq_block_size)
from .worker.block_manager import BlockManager  # noqa: F401
from .worker.kernels.kvcache_mgmt import store_kvcache  # noqa: F401
from .worker.kernels._deferred import enable_deferred_decode_append, flush as flush_pending_appends  # noqa: F401
from .worker.kernels.paged_attn import (decode_append_and_attend, decode_rope_append_and_attend,  # noqa: F401
                                        paged_attention)
from .worker.kernels.prefill_attn import prefill_attention, chunked_prefill_attention  # noqa: F401
from .worker.kernels.rotary_emb import (rotary_embedding_and_store_kvcache, rotary_embedding_inplace,  # noqa: F401
                                        rotary_tables)
from .elastic_pool import ElasticKVPool  # noqa: F401
from .kv_placement import allocate_kv_caches  # noqa: F401
from .vmm_pool import LayerArena, VmmKVPool  # noqa: F401
from .worker.swap import KVSwapper  # noqa: F401
from .worker.layers import attention_section  # noqa: F401
from . import swiftllm_c  # noqa: F401

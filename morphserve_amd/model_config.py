"""The model-shape fields the KV path reads, with the reference's accessor for the size of one
token's KV (MorphServe/model_config.py:5-46; pool sizing in MorphServe/worker/model.py:176-190 is
``num_blocks = bytes // (block_size * get_kvslot_size())``)."""
from __future__ import annotations

import json
import os

import torch


class LlamaModelConfig:
    """Built from the dict of a Hugging Face ``config.json`` of a LLaMA-family model; only the
    attention geometry is interpreted here, the remaining keys are kept as given in ``raw``."""

    def __init__(self, model_config: dict):
        if model_config.get("model_type", "llama") != "llama":
            raise ValueError(f"not a LLaMA-family config: model_type={model_config.get('model_type')!r}")
        self.raw = dict(model_config)
        self.num_layers = int(model_config["num_hidden_layers"])
        self.num_q_heads = int(model_config["num_attention_heads"])
        self.num_kv_heads = int(model_config.get("num_key_value_heads", self.num_q_heads))
        self.hidden_size = int(model_config["hidden_size"])
        self.head_dim = self.hidden_size // self.num_q_heads
        self.max_position_embeddings = int(model_config.get("max_position_embeddings", 4096))
        self.rope_theta = float(model_config.get("rope_theta", model_config.get("rotary_base", 10000)))
        scaling = model_config.get("rope_scaling", 1.0)
        self.rope_scaling = 1.0 if scaling is None else scaling

    def get_kvslot_size(self, dtype: torch.dtype = torch.float16) -> int:
        """Bytes of one token's K and V over all layers (model_config.py:36-40)."""
        return 2 * self.num_layers * self.num_kv_heads * self.head_dim * torch.empty((), dtype=dtype).element_size()

    def get_block_bytes(self, block_size: int, dtype: torch.dtype = torch.float16) -> int:
        """Bytes of one pool block, K and V together."""
        return block_size * self.get_kvslot_size(dtype)

    def num_blocks_that_fit(self, block_size: int, free_memory: int, total_memory: int,
                            gpu_mem_utilization: float, dtype: torch.dtype = torch.float16) -> int:
        """The pool size ``LlamaModel.profile_num_blocks`` arrives at once its forged prefill batch has run
        (MorphServe/worker/model.py:161-171): with ``free_memory, total_memory`` as ``torch.cuda.mem_get_info``
        reports them at the peak, ``floor((total * utilization - (total - free)) / block bytes)``;
        ``RuntimeError`` when the peak already exceeds the usable share."""
        peak = total_memory - free_memory
        usable = total_memory * gpu_mem_utilization
        if usable < peak:
            gb = 1024 ** 3
            raise RuntimeError(f"Peak memory {peak / gb:.2f} GB exceeds usable memory {usable / gb:.2f} GB "
                               f"({total_memory / gb:.2f} GB * {gpu_mem_utilization})")
        return int((usable - peak) // self.get_block_bytes(block_size, dtype))

    @staticmethod
    def load_from_model_path(model_path: str) -> "LlamaModelConfig":
        with open(os.path.join(model_path, "config.json"), "r", encoding="utf-8") as f:
            return LlamaModelConfig(json.load(f))

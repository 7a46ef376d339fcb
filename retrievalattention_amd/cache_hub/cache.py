"""KV_Cache base: shapes, the `context` counter and the free-memory estimate that decides
whether the GPU side of the cache is allocated before prefill (reference: cache_hub/cache.py)."""
import torch

GiB = 1024 ** 3


class KV_Cache:
    def __init__(self, layer_num, batch_size, max_length, num_key_value_heads, num_heads, head_dim, dtype,
                 layer_mapping, num_gpus, model_size):
        self.layer_num = layer_num
        self.batch_size = batch_size
        self.max_length = max_length
        self.kv_head = num_key_value_heads
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.dtype = dtype
        self.layer_mapping = layer_mapping
        self.context = 0
        self.num_gpus = num_gpus
        self.model_size = model_size
        # memory left for the cache while prefilling: total - weights (2 bytes/param, model_size
        # in billions) - activations of one max_length sequence (hidden, residual, qkv, 4 temps)
        total = num_gpus * torch.cuda.get_device_properties(0).total_memory / GiB
        per_token = (num_heads * 6 + (num_heads + 2 * num_key_value_heads)) * head_dim * 2
        self.free_memory = total - model_size * 2 - num_gpus * per_token * max_length / GiB

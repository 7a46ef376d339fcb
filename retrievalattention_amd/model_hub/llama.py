"""A Llama-shaped decoder around the wave-index attention: the caller side of the path
(reference: model_hub/LLM.py:32-208 layer_prefill / layer_decode / prefill_forward / decode_forward /
inference, model_hub/llama.py:222-346 the per-layer operators), with randomly initialised weights
(there are no checkpoints to load here).  Everything outside the attention is stock torch: RMSNorm,
the fused QKV projection, rotary embedding, the output projection and the SwiGLU MLP.

Two attention back-ends, as in the reference's attention_type switch:
  "RetroInfer"       the wave-index cache of this package (cache_hub.retroinfer_cache)
  "Full_Flash_Attn"  plain attention over a dense K/V cache (the baseline the reference compares with)

A whole decoded token (every layer) can be captured into one HIP graph and replayed token after
token: the wave-index cache is then built with device_positions=True, and the rotary position comes
from a device-side counter.
"""
import math
from dataclasses import dataclass

import torch

from ..attn_hub import retroinfer_prefill_attn, retroinfer_decode_attn
from ..cache_hub import retroinfer_cache


@dataclass
class LlamaShape:
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 128
    vocab_size: int = 128256
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5


class LlamaLayer:
    """Weights of one decoder layer (reference: model_hub/llama.py:15-47)."""

    def __init__(self, shape, dtype, device, gen):
        h, kv = shape.num_heads * shape.head_dim, shape.num_key_value_heads * shape.head_dim
        w = lambda o, i: (torch.randn(o, i, generator=gen, device=device, dtype=torch.float32) / math.sqrt(i)).to(dtype)
        self.wqkv = w(h + 2 * kv, shape.hidden_size)
        self.wo = w(shape.hidden_size, h)
        self.gate_up_proj = w(2 * shape.intermediate_size, shape.hidden_size)
        self.down_proj = w(shape.hidden_size, shape.intermediate_size)
        self.input_layernorm_weight = torch.ones(shape.hidden_size, dtype=dtype, device=device)
        self.post_attention_layernorm_weight = torch.ones(shape.hidden_size, dtype=dtype, device=device)


class DenseCache:
    """Plain K/V cache for the dense baseline: [B, max_length, Hkv, D] per layer."""

    def __init__(self, layer_num, batch_size, max_length, kv_heads, head_dim, dtype, device):
        shape = (batch_size, max_length, kv_heads, head_dim)
        self.k = [torch.zeros(shape, dtype=dtype, device=device) for _ in range(layer_num)]
        self.v = [torch.zeros(shape, dtype=dtype, device=device) for _ in range(layer_num)]
        self.layer_num = layer_num
        self.context = 0

    def prefill_update_kv_cache(self, q, k, v, layer_idx, batch_idx):
        n = k.shape[1]
        self.k[layer_idx][batch_idx, :n] = k[0]
        self.v[layer_idx][batch_idx, :n] = v[0]
        if layer_idx == self.layer_num - 1 and batch_idx == self.k[0].shape[0] - 1:
            self.context = n
        return k, v

    def decode_update_kv_cache(self, k, v, layer_idx):
        self.k[layer_idx][:, self.context] = k[:, 0]
        self.v[layer_idx][:, self.context] = v[:, 0]
        if layer_idx == self.layer_num - 1:
            self.context += 1
            return self.k[layer_idx][:, :self.context], self.v[layer_idx][:, :self.context]
        return self.k[layer_idx][:, :self.context + 1], self.v[layer_idx][:, :self.context + 1]


class LlamaModel:
    def __init__(self, shape, max_length, dtype=torch.bfloat16, device="cuda:0", seed=0):
        self.shape, self.max_length, self.dtype, self.device = shape, max_length, dtype, torch.device(device)
        self.num_layers = shape.num_layers
        self.num_heads, self.num_key_value_heads, self.head_dim = shape.num_heads, shape.num_key_value_heads, shape.head_dim
        self.hidden_size = shape.hidden_size
        gen = torch.Generator(device=self.device).manual_seed(seed)
        self.layers = [LlamaLayer(shape, dtype, self.device, gen) for _ in range(shape.num_layers)]
        self.embed_tokens = (torch.randn(shape.vocab_size, shape.hidden_size, generator=gen, device=self.device) * 0.5).to(dtype)
        self.lm_head = (torch.randn(shape.vocab_size, shape.hidden_size, generator=gen, device=self.device)
                        / math.sqrt(shape.hidden_size)).to(dtype)
        self.norm_weight = torch.ones(shape.hidden_size, dtype=dtype, device=self.device)
        inv_freq = 1.0 / (shape.rope_theta ** (torch.arange(0, shape.head_dim, 2, device=self.device).float() / shape.head_dim))
        freqs = torch.outer(torch.arange(max_length, device=self.device).float(), inv_freq)
        self.cos_cache, self.sin_cache = freqs.cos(), freqs.sin()          # [max_length, D/2] fp32
        self.position = torch.zeros(1, dtype=torch.int64, device=self.device)   # position of the token being decoded
        self.kv_cache = None
        self.attention_type = None

    # ------------------------------------------------------------------ operators (llama.py:222-346)
    def word_embedding(self, inputs_id):
        return torch.nn.functional.embedding(inputs_id, self.embed_tokens)

    def lm(self, hidden_states):
        return torch.matmul(hidden_states, self.lm_head.t()).float()

    def layernorm(self, hidden_states, weight):
        x = hidden_states.float()
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.shape.rms_eps)
        return (x * weight.float()).to(self.dtype)

    def wqkv(self, hidden_states, layer):
        qkv = torch.matmul(hidden_states, layer.wqkv.t())
        h, kv = self.num_heads * self.head_dim, self.num_key_value_heads * self.head_dim
        return qkv.split([h, kv, kv], dim=-1)

    def wo(self, attn_out, layer, bsz, seq_len):
        return torch.matmul(attn_out.reshape(bsz, seq_len, -1), layer.wo.t())

    def mlp(self, hidden_states, layer):
        gate, up = torch.matmul(hidden_states, layer.gate_up_proj.t()).chunk(2, dim=-1)
        return torch.matmul(torch.nn.functional.silu(gate) * up, layer.down_proj.t())

    def _rope(self, x, cos, sin):
        """x [B, S, H, D]; cos/sin [S, D/2] (or [1, D/2]); rotate-half convention."""
        x1, x2 = x.float().chunk(2, dim=-1)
        c, s = cos[None, :, None, :], sin[None, :, None, :]
        return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1).to(self.dtype)

    def position_embedd(self, query_states, key_states, positions):
        cos, sin = self.cos_cache.index_select(0, positions), self.sin_cache.index_select(0, positions)
        return self._rope(query_states, cos, sin), self._rope(key_states, cos, sin)

    # ------------------------------------------------------------------ cache
    def init_kv_cache(self, attention_type, batch_size, input_length, max_new_length, attn_config=None,
                      device_positions=False):
        """attn_config: n_centroids, n_segment, nprobe, max_compute_cluster_num, cache_cluster_num
        (reference: llama.py:154-211 reads them from config/<model>.json)."""
        self.attention_type = attention_type
        if attention_type == "Full_Flash_Attn":
            self.kv_cache = DenseCache(self.num_layers, batch_size, input_length + max_new_length,
                                       self.num_key_value_heads, self.head_dim, self.dtype, self.device)
            return
        if attention_type != "RetroInfer":
            raise ValueError(f"unknown attention type {attention_type}")
        c = attn_config
        self.kv_cache = retroinfer_cache(
            valid_start=[0] * batch_size, layer_num=self.num_layers, batch_size=batch_size,
            max_length=input_length + max_new_length, num_key_value_heads=self.num_key_value_heads,
            num_heads=self.num_heads, head_dim=self.head_dim, dtype=self.dtype,
            layer_mapping={str(l): str(self.device) for l in range(self.num_layers)}, max_new_length=max_new_length,
            static_pattern_start=c.get("static_pattern_start", 4), static_pattern_end=c.get("static_pattern_end", 64),
            core=c.get("core", 8), n_centroids=c["n_centroids"], n_segment=c.get("n_segment", 1), nprobe=c["nprobe"],
            max_compute_cluster_num=c["max_compute_cluster_num"], cache_unit_size=8,
            cache_cluster_num=c.get("cache_cluster_num", c["nprobe"] * 3), num_gpus=1, model_size=0,
            kv_residency=c.get("kv_residency", "device"), device_positions=device_positions)

    # ------------------------------------------------------------------ layers (LLM.py:32-127)
    def layer_prefill(self, layer_idx, start_bdx, hidden_states):
        bsz, seq_len, _ = hidden_states.shape
        layer = self.layers[layer_idx]
        residual = hidden_states
        hidden_states = self.layernorm(hidden_states, layer.input_layernorm_weight)
        q, k, v = self.wqkv(hidden_states, layer)
        q = q.view(bsz, seq_len, self.num_heads, self.head_dim)
        k = k.view(bsz, seq_len, self.num_key_value_heads, self.head_dim)
        v = v.view(bsz, seq_len, self.num_key_value_heads, self.head_dim).contiguous()
        q, k = self.position_embedd(q, k, torch.arange(seq_len, device=self.device))
        k, v = self.kv_cache.prefill_update_kv_cache(q, k.contiguous(), v, layer_idx, start_bdx)
        attn_out = retroinfer_prefill_attn(q, k, v, causal=True)
        if hasattr(self.kv_cache, "sync"):
            self.kv_cache.sync(layer_idx, start_bdx)
        hidden_states = residual + self.wo(attn_out, layer, bsz, seq_len)
        residual = hidden_states
        hidden_states = self.layernorm(hidden_states, layer.post_attention_layernorm_weight)
        return residual + self.mlp(hidden_states, layer)

    def decode_attention(self, q, k, v, layer_idx):
        if self.attention_type == "RetroInfer":
            return retroinfer_decode_attn(q, k, v, layer_idx, self.kv_cache)
        out = torch.nn.functional.scaled_dot_product_attention(
            q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), enable_gqa=True)
        return out.transpose(1, 2)

    def layer_decode(self, layer_idx, hidden_states):
        bsz, seq_len, _ = hidden_states.shape
        layer = self.layers[layer_idx]
        residual = hidden_states
        hidden_states = self.layernorm(hidden_states, layer.input_layernorm_weight)
        q, k, v = self.wqkv(hidden_states, layer)
        q = q.view(bsz, 1, self.num_heads, self.head_dim)
        k = k.view(bsz, 1, self.num_key_value_heads, self.head_dim)
        v = v.view(bsz, 1, self.num_key_value_heads, self.head_dim).contiguous()
        q, k = self.position_embedd(q, k, self.position)
        k, v = self.kv_cache.decode_update_kv_cache(k.contiguous(), v, layer_idx)
        attn_out = self.decode_attention(q.contiguous(), k, v, layer_idx)
        hidden_states = residual + self.wo(attn_out, layer, bsz, seq_len)
        residual = hidden_states
        hidden_states = self.layernorm(hidden_states, layer.post_attention_layernorm_weight)
        return residual + self.mlp(hidden_states, layer)

    # ------------------------------------------------------------------ forward passes (LLM.py:129-171)
    def prefill_forward(self, inputs_ids):
        bsz, seq_len = inputs_ids.shape
        last = torch.empty((bsz, 1, self.hidden_size), dtype=self.dtype, device=self.device)
        for b in range(bsz):
            hidden_states = self.word_embedding(inputs_ids[b:b + 1])
            for ldx in range(self.num_layers):
                hidden_states = self.layer_prefill(ldx, b, hidden_states)
            last[b] = hidden_states[0, -1:]
        if hasattr(self.kv_cache, "prepare_cache"):
            self.kv_cache.prepare_cache()
        self.position.fill_(seq_len)
        return self.lm(self.layernorm(last, self.norm_weight))

    def decode_forward(self, inputs_ids):
        """One token for every sequence: inputs_ids [B, 1] -> logits [B, 1, vocab].  Safe to capture:
        the position moves on by a device-side add."""
        hidden_states = self.word_embedding(inputs_ids)
        for ldx in range(self.num_layers):
            hidden_states = self.layer_decode(ldx, hidden_states)
        self.position.add_(1)
        return self.lm(self.layernorm(hidden_states, self.norm_weight))

    def generate(self, inputs_ids, max_new_length):
        """Greedy decoding (reference: LLM.py:174-208): returns [B, max_new_length] token ids."""
        logits = self.prefill_forward(inputs_ids)
        out = []
        tok = logits.argmax(-1)
        out.append(tok)
        for _ in range(max_new_length - 1):
            tok = self.decode_forward(tok).argmax(-1)
            out.append(tok)
        return torch.cat(out, dim=1)

"""attn_hub/retroinfer_attn.py of the reference: the two functions a model calls."""
import torch


def retroinfer_prefill_attn(query_states, key_states, value_states, causal):
    """Full causal attention over the prompt (reference: flash_attn_with_kvcache,
    attn_hub/retroinfer_attn.py:4-13).  Prefill attention is outside the wave-index path; it
    is served by the framework's fused SDPA.  Inputs [bsz, seq, heads, dim]."""
    q = query_states.transpose(1, 2)
    k = key_states.transpose(1, 2)
    v = value_states.transpose(1, 2)
    out = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=causal,
                                                           enable_gqa=k.shape[1] != q.shape[1])
    return out.transpose(1, 2)


def retroinfer_decode_attn(query_states, key_states, value_states, layer_idx, retroinfer_cache,
                           query_states_next=None):
    """attn_hub/retroinfer_attn.py:17-24."""
    return retroinfer_cache.compute(
        query_states.contiguous(), layer_idx,
        query_states_next.contiguous() if query_states_next is not None else None)

"""MI355X-native wave-index attention (RetroInfer's clustered KV-cache path).

    retrievalattention_amd.cache_hub.retroinfer_cache   the KV-cache class (reference API)
    retrievalattention_amd.attn_hub                     retroinfer_prefill_attn / retroinfer_decode_attn
    retrievalattention_amd.kernels                      retroinfer_kernels-compatible operators + fused ops
    retrievalattention_amd.build                        builds libretro_mi355.so with hipcc
"""

"""ctypes binding of libretro_mi355.so.  There is no fallback: if the library has not been
built (python -m retrievalattention_amd.build), importing the kernels raises."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libretro_mi355.so")

_lib = None

P, I, I64, F, SZ = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t

# name -> (restype, argtypes); mirrors include/retro_mi355.h
SIGNATURES = {
    "ri_status_string": (C.c_char_p, [I]),
    "ri_last_hip_error": (I, []),
    "ri_abi_version": (I, []),
    "ri_null_launch": (I, [P]),
    "ri_probe_stream_read": (I, [P, SZ, I, I, P, P]),
    "ri_batch_gemm_softmax": (I, [P, P, P, P, P, P, I, I, I, I, F, F, P]),
    "ri_batch_gemm_softmax_f16": (I, [P, P, P, P, P, P, I, I, I, I, F, F, P]),
    "ri_score_select_workspace_bytes": (SZ, [I, I, I]),
    "ri_score_select": (I, [P] * 13 + [I, P, I, I, I, I, I, I, I, F, P, SZ, P]),
    "ri_score_select_f16": (I, [P] * 13 + [I, P, I, I, I, I, I, I, I, F, P, SZ, P]),
    "ri_score_logits": (I, [P, P, P, I, I, I, F, P, SZ, P]),
    "ri_score_logits_f16": (I, [P, P, P, I, I, I, F, P, SZ, P]),
    "ri_flash_decoding_workspace_bytes": (SZ, [I, I]),
    "ri_attention_workspace_reset": (I, [P, SZ, P]),
    "ri_weighted_flash_decoding": (I, [P, P, P, P, P, P, P, P, P, I, I, I, I64, F, P, SZ, P]),
    "ri_weighted_flash_decoding_f16": (I, [P, P, P, P, P, P, P, P, P, I, I, I, I64, F, P, SZ, P]),
    "ri_wave_attention_workspace_bytes": (SZ, [I, I]),
    "ri_wave_attention": (I, [P, P, P, I64, I, P, P, P, I64, P, I, P, P, I, P, P, P, P, P, P, P, P, I, I, I, I, F, P, SZ, P]),
    "ri_wave_attention_f16": (I, [P, P, P, I64, I, P, P, P, I64, P, I, P, P, I, P, P, P, P, P, P, P, P, I, I, I, I, F, P, SZ, P]),
    "ri_wave_attention_part": (I, [P, P, P, I64, I, P, P, P, I64, P, I, I, I, P, P, P, P, P, P, P, P, P, P, I, I, I, I, F, P, SZ, P]),
    "ri_wave_attention_part_f16": (I, [P, P, P, I64, I, P, P, P, I64, P, I, I, I, P, P, P, P, P, P, P, P, P, P, I, I, I, I, F, P, SZ, P]),
    "ri_wave_attention_static_scratch_bytes": (SZ, []),
    "ri_wave_attention_static": (I, [P, P, P, I64, I, P, P, P, I64, P, I, P, P, I, P, P, P, P, P, P, P, P, I, I, I, I, F, P]),
    "ri_wave_attention_static_f16": (I, [P, P, P, I64, I, P, P, P, I64, P, I, P, P, I, P, P, P, P, P, P, P, P, I, I, I, I, F, P]),
    "ri_buffer_attention": (I, [P, P, P, I64, P, I, P, P, P, P, P, I, I, I, I, F, P, SZ, P]),
    "ri_buffer_attention_f16": (I, [P, P, P, I64, P, I, P, P, P, P, P, I, I, I, I, F, P, SZ, P]),
    "ri_lru_access_update": (I, [P, P, P, I, P, I, P, P, I, P, I, P, P, P] + [P] * 12 + [P, I, I, P] + [I] * 6 + [P]),
    "ri_gather_copy_vectors": (I, [P, P, P, P, P, P, P, I, I, I, I, I, I, P]),
    "ri_gather_copy_and_concat": (I, [P] * 17 + [I] * 7 + [P]),
    "ri_gather_copy_and_scatter": (I, [P] * 8 + [I] * 5 + [P]),
    "ri_kmeans_assign": (I, [P, P, P, I, I, I, I, I64, P]),
    "ri_kmeans_assign_f16": (I, [P, P, P, I, I, I, I, I64, P]),
    "ri_kmeans_workspace_bytes": (SZ, [I, I, I]),
    "ri_kmeans_build_lists": (I, [P, P, P, P, I, I, I, P, SZ, P]),
    "ri_kmeans_reduce_workspace_bytes": (SZ, [I, I, I]),
    "ri_kmeans_update": (I, [P, P, P, P, P, I, I, I, I, I64, I, P, SZ, P]),
    "ri_kmeans_update_f16": (I, [P, P, P, P, P, I, I, I, I, I64, I, P, SZ, P]),
    "ri_kmeans_value_sum": (I, [P, P, P, P, P, I, I, I, P, SZ, P]),
    "ri_kmeans_value_sum_f16": (I, [P, P, P, P, P, I, I, I, P, SZ, P]),
    "ri_permute_rows": (I, [P, P, P, I, I, I64, I64, P]),
    "ri_threadpool_create": (P, [I]),
    "ri_threadpool_create_pinned": (P, [I, I]),
    "ri_threadpool_pinned_workers": (I, [P]),
    "ri_threadpool_destroy": (None, [P]),
    "ri_wavebuf_create": (P, [I] * 10 + [P]),
    "ri_wavebuf_destroy": (None, [P]),
    "ri_wavebuf_set_indices": (I, [P] * 14),
    "ri_wavebuf_set_kv": (I, [P, P, P, I64, P, P, I64]),
    "ri_wavebuf_async_construction": (I, [P, P, P, I64, I]),
    "ri_wavebuf_construction_sync": (I, [P]),
    "ri_wavebuf_update_kv": (I, [P, P, P, I64, P, P, I, I64]),
    "ri_wavebuf_batch_access": (I, [P]),
    "ri_wavebuf_sync": (I, [P]),
    "ri_wavebuf_overflow_events": (I64, [P]),
}


def lib():
    """Loads the shared library once and declares every entry point."""
    global _lib
    if _lib is None:
        # torch ships its own HIP runtime; it has to be in the process first so that the library
        # binds to that one instead of bringing a second runtime with no device context
        import torch  # noqa: F401
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m retrievalattention_amd.build` "
                "(there is no CPU or PyTorch fallback for the wave-index kernels)")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status, what):
    if status != 0:
        l = lib()
        msg = l.ri_status_string(status).decode()
        if status == -2:
            msg += f" (hip error {l.ri_last_hip_error()})"
        raise RuntimeError(f"{what}: {msg}")

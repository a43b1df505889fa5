"""ctypes view of libwarpdecode_amd.so (the C ABI declared in include/warpdecode_amd.h).

Plumbing for the tests and the benchmark: device memory comes from torch tensors
(`t.data_ptr()`), the stream from `torch.cuda.current_stream().cuda_stream`.
There is no fallback: if the HIP library has not been built, loading raises.
"""
import ctypes as C
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libwarpdecode_amd.so")
HEADER = os.path.join(os.path.dirname(HERE), "include", "warpdecode_amd.h")

F32, F16, Q4_0, Q8_0, IQ4_NL, IQ3_S, IQ2_S = 0, 1, 2, 8, 20, 21, 22
Q6_K = 14
MOE_PRESELECTED, MOE_KEEP_EXPERT_OUT, MOE_STAGED = 1, 2, 4
MOE_ONLY_A, MOE_ONLY_B, MOE_ONLY_C, MOE_DRY, MOE_SPLIT_AB = 0x10, 0x20, 0x40, 0x80, 0x100
MOE_PER_LAYER = 0x200

vp, i32, f32, sz, u32 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint


class WdError(RuntimeError):
    pass


class GemvItem(C.Structure):
    """wd_gemv_item: one matrix of a batched exact-order Q8_0 GEMV."""
    _fields_ = [("d_w", vp), ("rows", i32), ("d_act_qs", vp), ("d_act_scales", vp), ("d_out", vp)]


class MoeLayer(C.Structure):
    _fields_ = [
        ("hidden", i32), ("expert_ffn", i32), ("n_experts", i32), ("top_k", i32),
        ("expert_scale", f32),
        ("gate_type", i32), ("up_type", i32), ("down_type", i32),
        ("router", vp),
        ("gate", vp), ("up", vp), ("down", vp),
        ("gate_stride", sz), ("up_stride", sz), ("down_stride", sz),
        ("slot_of_expert", vp), ("slot_pool", vp),
        ("slot_bytes", sz), ("slot_gate_bytes", sz), ("slot_up_bytes", sz),
        ("shared_gate_inp", vp),
        ("shared_gate", vp), ("shared_up", vp), ("shared_down", vp),
    ]


class FileMapping(C.Structure):
    _fields_ = [("start", C.c_uint64), ("end", C.c_uint64), ("file_offset", C.c_uint64), ("path", C.c_char * 4096)]


class GgufTensorInfo(C.Structure):
    _fields_ = [("name", C.c_char_p), ("n_dims", C.c_uint32), ("dims", C.c_uint64 * 4), ("type", C.c_uint32),
                ("relative_offset", C.c_uint64), ("bytes", C.c_uint64), ("data", vp)]


class ProfileSiteStat(C.Structure):
    _fields_ = [("calls", C.c_ulonglong), ("recorded", C.c_ulonglong), ("dropped", C.c_ulonglong),
                ("unreadable", C.c_ulonglong), ("device_ms", C.c_double), ("host_ms", C.c_double)]


class CacheStats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("accesses", "hits", "misses", "evictions", "bytes_copied", "slots",
                                          "slot_bytes", "resident")]


_SIGS = {
    "wd_init": (i32, [i32]),
    "wd_row_bytes": (sz, [i32, i32]),
    "wd_q8_0_quantize_f16": (i32, [vp, i32, vp, vp, vp]),
    "wd_q8_1_quantize_f32": (i32, [vp, i32, vp, vp, vp]),
    "wd_gemv_q8_0_q8_1_f32": (i32, [vp, i32, i32, vp, vp, vp, vp, vp]),
    "wd_convert_f16_to_f32": (i32, [vp, vp, sz, vp]),
    "wd_convert_f32_to_f16": (i32, [vp, vp, sz, vp]),
    "wd_gemv_q6_k_q8_k_f32": (i32, [vp, i32, i32, vp, vp, vp, vp, vp, vp]),
    "wd_file_mapping_of": (i32, [vp, C.POINTER(FileMapping)]),
    "wd_expert_cache_attach_mappings": (i32, [vp, i32, C.POINTER(i32)]),
    "wd_hc_combine_f32": (i32, [vp, vp, vp, i32, i32, i32, vp]),
    "wd_hc_combine_moe_f32": (i32, [vp, vp, vp, i32, vp, vp, i32, i32, i32, vp]),
    "wd_moe_layer_hc_f32": (i32, [C.POINTER(MoeLayer), vp, vp, vp, vp, i32, i32, vp, u32, vp]),
    "wd_tensor_bytes": (sz, [i32, i32, i32]),
    "wd_malloc": (i32, [C.POINTER(vp), sz]),
    "wd_free": (i32, [vp]),
    "wd_malloc_host": (i32, [C.POINTER(vp), sz]),
    "wd_free_host": (i32, [vp]),
    "wd_memcpy_h2d": (i32, [vp, vp, sz, vp]),
    "wd_memcpy_d2h": (i32, [vp, vp, sz, vp]),
    "wd_memcpy_d2d": (i32, [vp, vp, sz, vp]),
    "wd_memset": (i32, [vp, i32, sz, vp]),
    "wd_stream_create": (i32, [C.POINTER(vp)]),
    "wd_stream_destroy": (i32, [vp]),
    "wd_stream_sync": (i32, [vp]),
    "wd_device_sync": (i32, []),
    "wd_q8_k_quantize_f32": (i32, [vp, i32, vp, vp, vp, vp]),
    "wd_q8_0_quantize_f32": (i32, [vp, i32, vp, vp, vp]),
    "wd_router_gemv_f32": (i32, [vp, vp, vp, i32, i32, vp]),
    "wd_topk_softmax": (i32, [vp, i32, i32, f32, vp, vp, vp]),
    "wd_gemv_q8_k_f32": (i32, [i32, vp, i32, i32, vp, vp, vp, vp, vp]),
    "wd_gemv_q8_0_f32": (i32, [i32, vp, i32, i32, vp, vp, vp, vp, vp]),
    "wd_gemv_q8_0_batch_f32": (i32, [i32, vp, i32, i32, vp]),
    "wd_gemv_q8_k_experts_f32": (i32, [i32, vp, i32, i32, i32, vp, vp, vp, vp, vp]),
    "wd_gemv_q8_0_experts_f32": (i32, [i32, vp, i32, i32, i32, vp, vp, vp, vp, vp]),
    "wd_silu_mul_experts_f32": (i32, [vp, vp, i32, i32, vp]),
    "wd_weighted_accum_experts_f32": (i32, [vp, vp, vp, i32, i32, vp]),
    "wd_add_shared_f32": (i32, [vp, vp, vp, i32, vp]),
    "wd_moe_scratch_create": (i32, [C.POINTER(vp), i32, i32, i32, i32]),
    "wd_moe_scratch_destroy": (i32, [vp]),
    "wd_moe_scratch_enable_partials": (i32, [vp, i32, i32]),
    "wd_moe_scratch_trace": (vp, [vp, i32]),
    "wd_moe_scratch_trace_resident": (vp, [vp, i32, i32]),
    "wd_profile_enable": (i32, [i32]),
    "wd_profile_enabled": (i32, []),
    "wd_profile_begin": (i32, [i32, vp]),
    "wd_profile_end": (i32, [i32, vp]),
    "wd_profile_flush_token": (i32, []),
    "wd_profile_site": (i32, [i32, C.POINTER(ProfileSiteStat), C.POINTER(C.c_ulonglong)]),
    "wd_profile_site_name": (C.c_char_p, [i32]),
    "wd_profile_report": (sz, [C.c_char_p, sz]),
    "wd_profile_reset": (i32, []),
    "wd_moe_layer_f32": (i32, [C.POINTER(MoeLayer), vp, vp, vp, u32, vp]),
    "wd_moe_stack_cached_f32": (i32, [C.POINTER(MoeLayer), i32, vp, vp, vp, vp, vp, vp, f32, u32, vp]),
    "wd_moe_scratch_status": (i32, [vp]),
    "wd_moe_scratch_status_word": (vp, [vp]),
    "wd_moe_scratch_set_wait_limit": (i32, [vp, u32]),
    "wd_shared_expert_f32": (i32, [C.POINTER(MoeLayer), vp, vp, vp]),
    "wd_moe_stack_f32": (i32, [C.POINTER(MoeLayer), i32, vp, vp, vp, vp, f32, u32, vp]),
    "wd_moe_layer_noalloc_f32": (i32, [C.POINTER(MoeLayer), vp, vp, u32, vp]),
}
for _n in ("logits", "ids", "weights", "gate_up", "act", "act_qs", "act_scales", "expert_out", "accum", "down_f32",
           "shared_gate", "gate_up_partials", "down_partials"):
    _SIGS["wd_moe_scratch_" + _n] = (vp, [vp])

_OPTIONAL = {
    "wd_moe_layer_tokens_f32": (i32, [C.POINTER(MoeLayer), vp, vp, i32, C.POINTER(vp), u32, vp]),
    "wd_moe_layer_tokens_pairs_f32": (i32, [C.POINTER(MoeLayer), vp, vp, vp, i32, vp, vp, i32, C.POINTER(vp), u32, vp]),
    "wd_expert_cache_create": (i32, [C.POINTER(vp), sz, sz, sz, sz, i32, i32, i32]),
    "wd_expert_cache_destroy": (i32, [vp]),
    "wd_expert_cache_set_timing": (i32, [vp, i32]),
    "wd_expert_cache_register_layer": (i32, [vp, i32, vp, vp, vp]),
    "wd_expert_cache_acquire": (i32, [vp, i32, vp, i32, vp, vp]),
    "wd_expert_cache_slot_table": (vp, [vp, i32]),
    "wd_expert_cache_pool": (vp, [vp]),
    "wd_expert_cache_register_layer_strided": (i32, [vp, i32, vp, vp, vp, sz, sz, sz]),
    "wd_expert_cache_slot_of": (C.c_longlong, [vp, i32, i32]),
    "wd_expert_cache_add_shadow": (i32, [vp, i32, sz]),
    "wd_expert_cache_set_copy_kernel": (i32, [vp, i32]),
    "wd_expert_cache_set_read_ahead": (i32, [vp, i32, i32]),
    "wd_expert_cache_attach_file": (i32, [vp, vp, sz, i32, i32]),
    "wd_expert_cache_dump_json": (sz, [vp, C.c_char_p, sz]),
    "wd_gguf_open": (i32, [C.POINTER(vp), C.c_char_p]),
    "wd_gguf_close": (i32, [vp]),
    "wd_gguf_version": (C.c_uint32, [vp]),
    "wd_gguf_data_offset": (sz, [vp]),
    "wd_gguf_map_base": (vp, [vp]),
    "wd_gguf_map_bytes": (sz, [vp]),
    "wd_gguf_fd": (i32, [vp]),
    "wd_gguf_tensor_count": (C.c_longlong, [vp]),
    "wd_gguf_find": (C.c_longlong, [vp, C.c_char_p]),
    "wd_gguf_tensor": (i32, [vp, C.c_longlong, C.POINTER(GgufTensorInfo)]),
    "wd_gguf_meta_number": (i32, [vp, C.c_char_p, C.POINTER(C.c_double)]),
    "wd_gguf_meta_string": (C.c_char_p, [vp, C.c_char_p]),
    "wd_gguf_meta_array": (C.c_longlong, [vp, C.c_char_p, C.POINTER(C.c_uint32), C.POINTER(vp)]),
    "wd_expert_cache_get_stats": (i32, [vp, C.POINTER(CacheStats)]),
}


def declared_symbols():
    """Every function name include/warpdecode_amd.h declares."""
    txt = open(HEADER).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(wd_[a-z0-9_]+)\s*\(", txt)))


_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise WdError("libwarpdecode_amd.so is not built: run `python -m warpdecode_amd.build` "
                          "(there is no CPU fallback for the HIP kernels)")
        lib = C.CDLL(LIB_PATH)
        lib.wd_last_error.restype = C.c_char_p
        for name, (res, args) in list(_SIGS.items()) + list(_OPTIONAL.items()):
            fn = getattr(lib, name, None)
            if fn is None:
                if name in _SIGS:
                    raise WdError("libwarpdecode_amd.so does not export " + name)
                continue
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        raise WdError("wd error %d: %s" % (rc, load().wd_last_error().decode()))


def call(name, *args):
    check(getattr(load(), name)(*args))

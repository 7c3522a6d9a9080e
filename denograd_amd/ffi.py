"""ctypes bindings of libjsgrad_hip.so -- the same symbols a Deno `Deno.dlopen` binding would name
(the pattern of /root/reference/dawn/bindings.ts:5-8 and /root/reference/jsgrad/env/deno.ts:17).

The library is the product: nothing here falls back to a CPU path.  If the shared object is missing
or a call fails, a `HipError` is raised.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libjsgrad_hip.so")

F32, F16, BF16 = 0, 1, 2
W_F32, W_F16, W_I8, W_NF4 = 0, 1, 2, 3
PROF_KINDS = {"embed": 0, "rmsnorm": 1, "linear": 2, "qkv_rope": 3, "attn_decode": 4, "ffn_gate": 5, "argmax": 6, "decode_step": 7, "gemm": 8, "attn_prefill": 9, "attn_wo": 10, "read_probe": 11, "sample": 12}


class HipError(RuntimeError):
    pass


_vp, _i32, _f32, _sz, _u64 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint64
_pp = C.POINTER(C.c_void_p)

# name -> (argtypes, restype); every entry point declared in include/jsgrad_hip.h
SIGNATURES: dict[str, tuple[list, object]] = {
    "jsgrad_hip_init": ([_i32], _i32),
    "jsgrad_hip_last_error": ([], C.c_char_p),
    "jsgrad_hip_device_name": ([C.c_char_p, _sz], _i32),
    "jsgrad_hip_cu_count": ([C.POINTER(_i32)], _i32),
    "jsgrad_hip_malloc": ([_sz, _pp], _i32),
    "jsgrad_hip_free": ([_vp], _i32),
    "jsgrad_hip_free_cache": ([], _i32),
    "jsgrad_hip_mem_info": ([C.POINTER(_sz), C.POINTER(_sz)], _i32),
    "jsgrad_hip_copyin": ([_vp, _vp, _sz], _i32),
    "jsgrad_hip_copyout": ([_vp, _vp, _sz], _i32),
    "jsgrad_hip_copy": ([_vp, _vp, _sz], _i32),
    "jsgrad_hip_memset": ([_vp, _i32, _sz], _i32),
    "jsgrad_hip_sync": ([], _i32),
    "jsgrad_hip_module_load": ([_vp, _sz, _pp], _i32),
    "jsgrad_hip_module_unload": ([_vp], _i32),
    "jsgrad_hip_module_get": ([_vp, C.c_char_p, _pp], _i32),
    "jsgrad_hip_launch": ([_vp, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), _pp, _i32, C.POINTER(C.c_int32), _i32, _i32, C.POINTER(C.c_double)], _i32),
    "jsgrad_hip_event_create": ([_pp], _i32),
    "jsgrad_hip_event_record": ([_vp], _i32),
    "jsgrad_hip_event_elapsed_ms": ([_vp, _vp, C.POINTER(_f32)], _i32),
    "jsgrad_hip_event_destroy": ([_vp], _i32),
    "jsgrad_hip_profile": ([_i32], _i32),
    "jsgrad_hip_profile_read": ([_i32, C.POINTER(_i32), C.POINTER(C.c_double)], _i32),
    "jsgrad_hip_graph_begin": ([], _i32),
    "jsgrad_hip_graph_end": ([_pp], _i32),
    "jsgrad_hip_graph_launch": ([_vp], _i32),
    "jsgrad_hip_graph_destroy": ([_vp], _i32),
    "jsgrad_hip_rope_table": ([_vp, _i32, _i32, _f32, _i32], _i32),
    "jsgrad_hip_embed": ([_i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32], _i32),
    "jsgrad_hip_rmsnorm": ([_vp, _vp, _vp, _i32, _f32, _i32], _i32),
    "jsgrad_hip_linear": ([_i32, _vp, _vp, _i32, _i32, _vp, _vp, _vp, _f32, _vp, _i32], _i32),
    "jsgrad_hip_qkv_rope": ([_i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32], _i32),
    "jsgrad_hip_attn_workspace_bytes": ([_i32, _i32, _i32], _sz),
    "jsgrad_hip_attn_decode": ([_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32], _i32),
    "jsgrad_hip_attn_decode_status": ([_vp, _i32, _i32, _i32, C.POINTER(_i32)], _i32),
    "jsgrad_hip_attn_decode_static_max_bytes": ([], _sz),
    "jsgrad_hip_attn_decode_static": ([_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32], _i32),
    "jsgrad_hip_attn_decode_static_status": ([C.POINTER(_i32)], _i32),
    "jsgrad_hip_attn_wo_workspace_bytes": ([_i32, _i32, _i32], _sz),
    "jsgrad_hip_attn_wo": ([_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _vp, _i32, _vp, _vp, _i32], _i32),
    "jsgrad_hip_attn_wo_status": ([_vp, C.POINTER(_i32)], _i32),
    "jsgrad_hip_attn_wo_items": ([_i32, _i32], _i32),
    "jsgrad_hip_attn_wo_fits": ([_i32, _i32, _i32, _i32, _i32, _i32, C.POINTER(_i32), C.POINTER(_i32)], _i32),
    "jsgrad_hip_ffn_gate": ([_i32, _vp, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _i32, _i32, _i32], _i32),
    "jsgrad_hip_argmax": ([_vp, _i32, _vp, _vp, _i32, _i32, _i32], _i32),
    "jsgrad_hip_embed_rows": ([_i32, _vp, _vp, _vp, _i32, _vp, _i32, _i32], _i32),
    "jsgrad_hip_rmsnorm_rows": ([_vp, _vp, _vp, _i32, _i32, _f32], _i32),
    "jsgrad_hip_gemm": ([_i32, _vp, _vp, _i32, _i32, _vp, _i32, _vp, _vp], _i32),
    "jsgrad_hip_gemm_qkv_rope": ([_i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32], _i32),
    "jsgrad_hip_gemm_ffn_gate": ([_i32, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _i32, _i32], _i32),
    "jsgrad_hip_attn_prefill": ([_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32], _i32),
    "jsgrad_hip_attn_batch_workspace_bytes": ([_i32, _i32, _i32, _i32], _sz),
    "jsgrad_hip_attn_decode_batch": ([_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32], _i32),
    "jsgrad_hip_argmax_rows": ([_vp, _i32, _i32, _vp], _i32),
    "jsgrad_hip_step_workspace_bytes": ([_i32, _i32, _i32], _sz),
    "jsgrad_hip_decode_step": ([_vp], _i32),
    "jsgrad_hip_step_status": ([_vp, C.POINTER(_i32)], _i32),
    "jsgrad_hip_stream_workspace_bytes": ([_i32, _i32, _i32], _sz),
    "jsgrad_hip_stream_step": ([_vp], _i32),
    "jsgrad_hip_stream_status": ([_vp, C.POINTER(_i32)], _i32),
    "jsgrad_hip_read_probe": ([_vp, _sz, _vp], _i32),
    "jsgrad_hip_sample_workspace_bytes": ([_i32], _sz),
    "jsgrad_hip_sample": ([_vp, _i32, _i32, C.c_double, _i32, C.c_double, C.c_double, C.c_double, _vp, _vp, _vp, _vp, _i32, _i32, _vp], _i32),
    "jsgrad_hip_ggml_nbytes": ([_i32, _sz], _sz),
    "jsgrad_hip_ggml_dequant": ([_i32, _vp, _sz, _vp], _i32),
    "jsgrad_hip_cast": ([_vp, _i32, _vp, _i32, _sz], _i32),
    "jsgrad_hip_hf_permute": ([_vp, _vp, _i32, _i32, _i32], _i32),
    "jsgrad_hip_int8_quantize": ([_vp, _i32, _i32, _vp, _vp, _i32], _i32),
    "jsgrad_hip_int8_dequant": ([_vp, _vp, _i32, _i32, _vp], _i32),
    "jsgrad_hip_nf4_quantize": ([_vp, _sz, _vp, _vp, _i32], _i32),
    "jsgrad_hip_nf4_dequant": ([_vp, _vp, _sz, _vp], _i32),
    "jsgrad_hip_randn": ([_vp, _sz, _i32, _u64, _f32], _i32),
    "jsgrad_hip_fill": ([_vp, _sz, _i32, _f32], _i32),
}



class LayerDesc(C.Structure):
    """jsgrad_hip_layer_t"""
    _fields_ = [(n, C.c_void_p) for n in ("wq", "wk", "wv", "wo", "w1", "w2", "w3", "sq", "sk", "sv", "so", "s1", "s2", "s3",
                                           "attention_norm", "ffn_norm", "cache_k", "cache_v")]


class StepDesc(C.Structure):
    """jsgrad_hip_step_t"""
    _fields_ = ([("layers", C.c_void_p)] + [(n, C.c_int) for n in ("n_layers", "dim", "hidden", "n_heads", "n_kv_heads", "head_dim", "vocab", "max_context")]
                + [("eps", C.c_float)] + [(n, C.c_int) for n in ("kind", "out_kind", "embed_kind", "act")]
                + [(n, C.c_void_p) for n in ("tok_emb", "tok_scale", "out_w", "out_s", "final_norm", "rope_table", "state", "tokens_out")]
                + [("tokens_cap", C.c_int)] + [(n, C.c_void_p) for n in ("h", "h2", "q", "attn", "g", "logits", "workspace", "trace")])


_lib: C.CDLL | None = None


def load() -> C.CDLL:
    """dlopen the library and type every entry point.  No GPU call is made."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipError(f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                           "(make -C denograd_amd/csrc); there is no CPU fallback")
        lib = C.CDLL(LIB_PATH)
        for name, (args, res) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = args, res
        _lib = lib
    return _lib


def check(status: int) -> None:
    if status != 0:
        raise HipError(load().jsgrad_hip_last_error().decode(errors="replace"))

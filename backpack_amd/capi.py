"""ctypes binding of libbpk_kquant.so (include/bpk_kquant.h).

Device pointers are passed as integers (e.g. torch.Tensor.data_ptr()).  The
library is loaded from the package directory; it is never built implicitly and
loading fails loudly when it is missing."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbpk_kquant.so")

Q4_K = 12
Q5_K = 13
Q6_K = 14

FAMILY_AUTO, FAMILY_GENERIC, FAMILY_GEMV_ROWS, FAMILY_MFMA_SMALL, FAMILY_MFMA_GEMM = range(5)


class BpkError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"bpk error {code}: {msg}")
        self.code = code


class WeightDesc(C.Structure):
    _fields_ = [("type", C.c_int), ("N", C.c_uint32), ("K", C.c_uint32),
                ("n_blocks", C.c_uint32), ("row_stride_words", C.c_uint32),
                ("data", C.c_void_p), ("bytes", C.c_size_t)]


class Fusion(C.Structure):
    _fields_ = [("prologue", C.c_int), ("norm_w", C.c_void_p), ("eps", C.c_float), ("residual", C.c_void_p),
                ("epilogue", C.c_int)]


class ChainOp(C.Structure):
    _fields_ = [("type", C.c_int), ("X", C.c_void_p), ("W", C.c_void_p), ("bias", C.c_void_p), ("Y", C.c_void_p),
                ("N", C.c_uint32), ("K", C.c_uint32), ("n_blocks", C.c_uint32), ("row_stride_words", C.c_uint32),
                ("y_offset", C.c_uint32), ("fusion", Fusion)]


PRO_NONE, PRO_RMS_NORM, PRO_SILU_MUL, PRO_GELU_MUL = range(4)
EPI_NONE, EPI_SILU_MUL, EPI_GELU_MUL = 0, 2, 3


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("type", C.c_uint32), ("n_dims", C.c_uint32), ("dims", C.c_uint64 * 4),
                ("offset", C.c_uint64), ("bytes", C.c_uint64), ("data", C.c_void_p)]


class ModelConfig(C.Structure):
    """bpk_model_config: the reference's ModelConfig (runtime/gguf_loader.h:164-218) as a flat record."""
    _fields_ = [("arch", C.c_char * 64),
                ("n_layer", C.c_uint32), ("n_head", C.c_uint32), ("n_kv_heads", C.c_uint32), ("n_embd", C.c_uint32),
                ("intermediate_size", C.c_uint32), ("n_vocab", C.c_uint32), ("head_dim", C.c_uint32),
                ("kv_head_dim", C.c_uint32), ("rms_norm_eps", C.c_float), ("rope_theta", C.c_float),
                ("tie_word_embeddings", C.c_int), ("has_qk_norm", C.c_int), ("activation", C.c_int),
                ("embedding_scale", C.c_float), ("logit_softcap", C.c_float), ("sliding_window", C.c_uint32),
                ("n_layer_attn_types", C.c_uint32), ("has_sandwich_norm", C.c_int), ("ple_size", C.c_uint32),
                ("shared_kv_layers", C.c_uint32), ("has_mtp", C.c_int), ("mtp_num_layers", C.c_uint32),
                ("num_experts", C.c_uint32), ("num_experts_per_tok", C.c_uint32), ("moe_intermediate_size", C.c_uint32),
                ("moe_shared_intermediate_size", C.c_uint32), ("ssm_inner_size", C.c_uint32),
                ("ssm_state_size", C.c_uint32), ("ssm_conv_kernel", C.c_uint32), ("ssm_group_count", C.c_uint32),
                ("ssm_time_step_rank", C.c_uint32), ("full_attention_interval", C.c_uint32),
                ("rope_sections", C.c_int32 * 4)]


_SIGS = {
    "bpk_version": (C.c_int, []),
    "bpk_gemm_plan": (C.c_int, [C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.POINTER(C.c_int),
                                C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "bpk_last_error": (C.c_char_p, []),
    "bpk_last_kernel": (C.c_char_p, []),
    "bpk_force_kernel": (C.c_int, [C.c_int]),
    "bpk_set_option": (C.c_int, [C.c_char_p, C.c_int]),
    "bpk_init": (C.c_int, [C.c_int]),
    "bpk_shutdown": (C.c_int, []),
    "bpk_kq_layout": (C.c_int, [C.c_int, C.c_uint32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "bpk_kq_pack_host": (C.c_int, [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p]),
    "bpk_weight_create": (C.c_int, [C.c_int, C.c_uint32, C.c_uint32, C.POINTER(C.c_void_p),
                                    C.POINTER(C.c_uint32), C.POINTER(C.c_void_p)]),
    "bpk_weight_describe": (C.c_int, [C.c_void_p, C.POINTER(WeightDesc)]),
    "bpk_weight_destroy": (C.c_int, [C.c_void_p]),
    "bpk_gguf_open": (C.c_int, [C.c_char_p, C.POINTER(C.c_void_p)]),
    "bpk_gguf_close": (C.c_int, [C.c_void_p]),
    "bpk_gguf_info": (C.c_int, [C.c_void_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
                                C.POINTER(C.c_uint64)]),
    "bpk_gguf_tensor_at": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(GgufTensor)]),
    "bpk_gguf_find_tensor": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(GgufTensor)]),
    "bpk_gguf_has_key": (C.c_int, [C.c_void_p, C.c_char_p]),
    "bpk_gguf_key_type": (C.c_int, [C.c_void_p, C.c_char_p]),
    "bpk_gguf_get_u32": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint32, C.POINTER(C.c_uint32)]),
    "bpk_gguf_get_f32": (C.c_int, [C.c_void_p, C.c_char_p, C.c_float, C.POINTER(C.c_float)]),
    "bpk_gguf_get_bool": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int, C.POINTER(C.c_int)]),
    "bpk_gguf_get_string": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t, C.POINTER(C.c_size_t)]),
    "bpk_gguf_array_len": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32)]),
    "bpk_gguf_array_string": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_void_p, C.c_size_t,
                                        C.POINTER(C.c_size_t)]),
    "bpk_gguf_model_config": (C.c_int, [C.c_void_p, C.POINTER(ModelConfig), C.c_void_p, C.c_uint32]),
    "bpk_gguf_array_data": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_uint64),
                                      C.POINTER(C.c_uint32)]),
    "bpk_gguf_weight_create": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), C.c_uint32, C.POINTER(C.c_void_p)]),
    "bpk_kq_matmul": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p]),
    "bpk_kq_matmul_fused_workspace_bytes": (C.c_size_t, [C.c_uint32, C.c_uint32, C.c_uint32]),
    "bpk_kq_matmul_fused": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                      C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32,
                                      C.POINTER(Fusion), C.c_void_p, C.c_size_t, C.c_void_p]),
    "bpk_kq_matmul_bf16": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                     C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p]),
    "bpk_prefill_rows_bf16": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_float, C.c_uint32, C.c_uint32,
                                        C.c_void_p, C.c_void_p]),
    "bpk_kq_dequant_rows": (C.c_int, [C.c_int, C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32, C.c_uint32,
                                      C.c_void_p, C.c_void_p]),
    "bpk_kq_moe_matmul": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                    C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32,
                                    C.c_int, C.c_void_p]),
    "bpk_chain_create": (C.c_int, [C.POINTER(ChainOp), C.c_uint32, C.POINTER(C.c_void_p)]),
    "bpk_chain_run": (C.c_int, [C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p]),
    "bpk_chain_status": (C.c_int, [C.c_void_p]),
    "bpk_chain_reset": (C.c_int, [C.c_void_p]),
    "bpk_chain_destroy": (C.c_int, [C.c_void_p]),
    "bpk_chain_trace": (C.c_int, [C.c_void_p]),
    "bpk_argmax_rows": (C.c_int, [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "bpk_argmax_rows_static": (C.c_int, [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p,
                                         C.c_void_p]),
    "bpk_kq_matmul_argmax": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32,
                                       C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "bpk_moe_topk_softmax": (C.c_int, [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int, C.c_void_p, C.c_void_p,
                                       C.c_void_p]),
    "bpk_moe_route": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int,
                                C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "bpk_kq_moe_ffn_scratch_bytes": (C.c_size_t, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32]),
    "bpk_kq_moe_ffn": (C.c_int, [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                 C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32,
                                 C.c_uint32, C.c_uint32, C.c_void_p, C.c_size_t, C.c_void_p]),
}

_lib = None


def exported_names():
    return sorted(_SIGS)


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: build it with `python -m backpack_amd.build`")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise BpkError(rc, lib().bpk_last_error().decode())


def layout(type_: int, K: int):
    nb, rs = C.c_uint32(), C.c_uint32()
    check(lib().bpk_kq_layout(type_, K, C.byref(nb), C.byref(rs)))
    return nb.value, rs.value


def last_kernel() -> str:
    return lib().bpk_last_kernel().decode()


def force_kernel(family: int) -> None:
    check(lib().bpk_force_kernel(family))


def set_option(name: str, value: int) -> None:
    check(lib().bpk_set_option(name.encode(), value))


def gemm_plan(type_: int, M: int, N: int, K: int, compute_units: int = 256):
    """(form, share, rows_first) of the bf16 dequant-GEMM for a shape: host arithmetic, no device needed."""
    form, share, first = C.c_int(), C.c_uint32(), C.c_uint32()
    check(lib().bpk_gemm_plan(type_, M, N, K, compute_units, C.byref(form), C.byref(share), C.byref(first)))
    return form.value, share.value, first.value

"""ctypes binding of libautograph_hip.so (the C ABI declared in include/autograph_hip.h).

There is no CPU fallback: if the shared library is missing or fails to load, importing
this module raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libautograph_hip.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
        "(or __graft_entry__.build()); autograph_amd has no fallback path"
    )
lib = C.CDLL(LIB_PATH)

i64 = C.c_int64
ptr = C.c_void_p
f32 = C.c_float

_GEMM = [i64, i64, i64, f32, ptr, i64, i64, i64, ptr, i64, i64, i64, f32, ptr, i64, i64, i64]
_GEMM_B = [i64, i64, i64, i64, f32, ptr, i64, i64, i64, i64, ptr, i64, i64, i64, i64, f32, ptr, i64, i64, i64, i64,
           ptr, i64, i64, C.c_int]
_CONV = [ptr, ptr] + [i64] * 12
_POOL = [ptr, ptr] + [i64] * 7

SIGNATURES = {
    "agh_init": ([C.c_int], C.c_int),
    "agh_shutdown": ([], C.c_int),
    "agh_last_error_string": ([], C.c_char_p),
    "agh_device_info": ([C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_size_t)], C.c_int),
    "agh_malloc": ([C.POINTER(ptr), C.c_size_t], C.c_int),
    "agh_free": ([ptr], C.c_int),
    "agh_cache_release": ([], C.c_int),
    "agh_cache_stats": ([C.POINTER(C.c_size_t)] * 3, C.c_int),
    "agh_workspace_stats": ([C.POINTER(C.c_size_t)] * 2, C.c_int),
    "agh_memcpy_h2d": ([ptr, ptr, C.c_size_t], C.c_int),
    "agh_memcpy_d2h": ([ptr, ptr, C.c_size_t], C.c_int),
    "agh_memcpy_d2d": ([ptr, ptr, C.c_size_t], C.c_int),
    "agh_memcpy_d2h_async": ([ptr, ptr, C.c_size_t], C.c_int),
    "agh_host_alloc": ([C.POINTER(ptr), C.c_size_t], C.c_int),
    "agh_host_free": ([ptr], C.c_int),
    "agh_branch_begin": ([], C.c_int),
    "agh_branch_end": ([], C.c_int),
    "agh_branch_join": ([], C.c_int),
    "agh_graph_begin": ([], C.c_int),
    "agh_graph_end": ([C.POINTER(ptr)], C.c_int),
    "agh_graph_launch": ([ptr], C.c_int),
    "agh_graph_destroy": ([ptr], C.c_int),
    "agh_memset": ([ptr, C.c_int, C.c_size_t], C.c_int),
    "agh_sync": ([], C.c_int),
    "agh_stream": ([], ptr),
    "agh_event_create": ([C.POINTER(ptr)], C.c_int),
    "agh_event_destroy": ([ptr], C.c_int),
    "agh_event_record": ([ptr], C.c_int),
    "agh_event_elapsed_ms": ([ptr, ptr, C.POINTER(f32)], C.c_int),
    "agh_gemm_f32": (_GEMM, C.c_int),
    "agh_gemm_bf16": (_GEMM, C.c_int),
    "agh_gemm_bf16_noalloc": (_GEMM, C.c_int),
    "agh_gemm_f32_bias_act": (_GEMM + [ptr, i64, i64, C.c_int], C.c_int),
    "agh_gemm_bf16_bias_act": (_GEMM + [ptr, i64, i64, C.c_int], C.c_int),
    "agh_gemm_f32_batched": (_GEMM_B, C.c_int),
    "agh_gemm_bf16_batched": (_GEMM_B, C.c_int),
    "agh_im2col_conv2_f32": (_CONV, C.c_int),
    "agh_im2col_conv2_bf16": (_CONV, C.c_int),
    "agh_col2im_conv2_f32": (_CONV, C.c_int),
    "agh_col2im_conv2_bf16": (_CONV, C.c_int),
    "agh_conv2_direct_f32": ([ptr, ptr, ptr, ptr] + [i64] * 13 + [C.c_int, C.c_int], C.c_int),
    "agh_conv2_direct_bf16": ([ptr, ptr, ptr, ptr] + [i64] * 13 + [C.c_int, C.c_int], C.c_int),
    "agh_lenet5_forward_f32": ([ptr] * 8 + [i64], C.c_int),
    "agh_lenet5_forward_bf16": ([ptr] * 8 + [i64], C.c_int),
    "agh_lenet5_forward_train_f32": ([ptr] * 16 + [i64], C.c_int),
    "agh_lenet5_forward_train_bf16": ([ptr] * 16 + [i64], C.c_int),
    "agh_lenet5_backward_f32": ([ptr, ptr, C.c_float] + [ptr] * 13 + [i64], C.c_int),
    "agh_lenet5_backward_bf16": ([ptr, ptr, C.c_float] + [ptr] * 13 + [i64], C.c_int),
    "agh_lenet5_dense_weight_grads_f32": ([ptr] * 13 + [i64], C.c_int),
    "agh_lenet5_dense_weight_grads_bf16": ([ptr] * 13 + [i64], C.c_int),
    "agh_lenet5_conv_weight_grads_f32": ([ptr] * 6 + [i64], C.c_int),
    "agh_lenet5_conv_weight_grads_bf16": ([ptr] * 6 + [i64], C.c_int),
    "agh_max_pool2_f32": (_POOL, C.c_int),
    "agh_max_pool2_bf16": (_POOL, C.c_int),
    "agh_max_pool2_backward_f32": (_POOL, C.c_int),
    "agh_max_pool2_backward_bf16": (_POOL, C.c_int),
    "agh_relu_f32": ([ptr, ptr, i64], C.c_int),
    "agh_relu_bf16": ([ptr, ptr, i64], C.c_int),
    "agh_conv2_backward_input_f32": ([ptr, ptr, ptr] + [i64] * 13, C.c_int),
    "agh_conv2_backward_input_bf16": ([ptr, ptr, ptr] + [i64] * 13, C.c_int),
    "agh_relu_max_pool2_f32": ([ptr, ptr] + [i64] * 7, C.c_int),
    "agh_relu_max_pool2_bf16": ([ptr, ptr] + [i64] * 7, C.c_int),
    "agh_max_pool2_relu_backward_f32": ([ptr, ptr, ptr] + [i64] * 8 + [C.c_int], C.c_int),
    "agh_max_pool2_relu_backward_bf16": ([ptr, ptr, ptr] + [i64] * 8 + [C.c_int], C.c_int),
    "agh_relu_backward_f32": ([ptr, ptr, ptr, i64], C.c_int),
    "agh_relu_backward_bf16": ([ptr, ptr, ptr, i64], C.c_int),
    "agh_assign_f32": ([ptr] + [i64] * 5 + [ptr] + [i64] * 9, C.c_int),
    "agh_assign_bf16": ([ptr] + [i64] * 5 + [ptr] + [i64] * 9, C.c_int),
    "agh_scaled_add_f32": ([ptr, f32, ptr, i64], C.c_int),
    "agh_scaled_add_bf16": ([ptr, f32, ptr, i64], C.c_int),
    "agh_scaled_add_strided_f32": ([ptr] + [i64] * 5 + [f32, ptr] + [i64] * 9, C.c_int),
    "agh_scaled_add_strided_bf16": ([ptr] + [i64] * 5 + [f32, ptr] + [i64] * 9, C.c_int),
    "agh_sgd_momentum_f32": ([ptr, ptr, f32, f32, ptr, i64], C.c_int),
    "agh_sgd_momentum_bf16": ([ptr, ptr, f32, f32, ptr, i64], C.c_int),
    "agh_sum_axis0_f32": ([ptr, ptr, i64, i64], C.c_int),
    "agh_sum_axis0_bf16": ([ptr, ptr, i64, i64], C.c_int),
    "agh_cross_entropy_loss_f32": ([ptr, ptr, i64, i64, ptr], C.c_int),
    "agh_cross_entropy_loss_bf16": ([ptr, ptr, i64, i64, ptr], C.c_int),
    "agh_cross_entropy_backward_f32": ([ptr, ptr, f32, ptr, i64, i64], C.c_int),
    "agh_cross_entropy_backward_bf16": ([ptr, ptr, f32, ptr, i64, i64], C.c_int),
    "agh_accuracy_f32": ([ptr, ptr, i64, i64, ptr], C.c_int),
    "agh_accuracy_bf16": ([ptr, ptr, i64, i64, ptr], C.c_int),
}

for _name, (_args, _res) in SIGNATURES.items():
    _f = getattr(lib, _name)  # AttributeError here means the library does not export the symbol
    _f.argtypes = _args
    _f.restype = _res


class AghError(RuntimeError):
    """A non-zero status from the C ABI (the reference returns anyhow::Error here)."""

    def __init__(self, code, msg):
        super().__init__(f"[{code}] {msg}")
        self.code = code


def check(code):
    if code != 0:
        raise AghError(code, lib.agh_last_error_string().decode(errors="replace"))

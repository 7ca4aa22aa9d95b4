"""ctypes binding of libzant_hip.so: loads the library (loudly failing when it is missing), declares the
prototype of every entry point in include/zant_hip.h and wraps the context."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
lib_path = os.path.join(_HERE, "libzant_hip.so")

if not os.path.exists(lib_path):
    raise ImportError(
        f"{lib_path} is not built. Run `python z-ant_amd/build.py` (hipcc, gfx950). "
        "This backend has no CPU fallback.")

# torch ships its own copy of the HIP runtime.  Two runtimes in one process do not share the device (the second
# one to initialise reports "no ROCm-capable device"), so torch's must be mapped before the library's dependency
# on libamdhip64.so is resolved: the loader then binds the library to the copy that is already there.
import torch  # noqa: E402,F401

lib = C.CDLL(lib_path)

c_i64p = C.POINTER(C.c_int64)
vp, i64, i32, f32, u8, sz = C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_uint8, C.c_size_t

# name -> (restype, argtypes); mirrors include/zant_hip.h one to one
PROTOTYPES = {
    "zant_hip_ctx_create": (i32, [C.POINTER(vp), i32, vp]),
    "zant_hip_ctx_destroy": (None, [vp]),
    "zant_hip_sync": (i32, [vp]),
    "zant_hip_status_name": (C.c_char_p, [i32]),
    "zant_hip_last_error": (C.c_char_p, [vp]),
    "zant_hip_version": (C.c_char_p, []),
    "setLogFunctionC": (None, [vp]),
    "setLogFunction": (None, [vp]),
    "zant_hip_arena_reserve": (i32, [vp, sz]),
    "zant_hip_arena_ptr": (vp, [vp, sz]),
    "zant_hip_arena_size": (sz, [vp]),
    "zant_hip_malloc": (i32, [vp, C.POINTER(vp), sz]),
    "zant_hip_free": (i32, [vp, vp]),
    "zant_hip_upload": (i32, [vp, vp, vp, sz]),
    "zant_hip_download": (i32, [vp, vp, vp, sz]),
    "zant_hip_memset": (i32, [vp, vp, i32, sz]),
    "zant_hip_timer_start": (i32, [vp]),
    "zant_hip_timer_stop": (i32, [vp, C.POINTER(f32)]),
    "zant_hip_kernel_timing": (i32, [vp, i32]),
    "zant_hip_kernel_ms": (i32, [vp, C.POINTER(f32)]),
    "zant_hip_kernel_name": (C.c_char_p, [vp]),
    "zant_hip_conv2d_f32": (i32, [vp, vp, c_i64p, vp, c_i64p, vp, vp, c_i64p, c_i64p, i32, c_i64p, i32, c_i64p, i32,
                                  i64, C.c_char_p, i32]),
    "zant_hip_conv2d_f32_static": (i32, [vp, vp, c_i64p, vp, c_i64p, vp, vp, c_i64p, c_i64p, i32, c_i64p, i32, c_i64p,
                                         i32, i64, C.c_char_p, i32]),
    "zant_hip_conv2d_f32_prepack": (i32, [vp, c_i64p, vp, c_i64p, vp, c_i64p, c_i64p, i32, c_i64p, i32, c_i64p, i32, i64,
                                          C.c_char_p, i32, i32, C.POINTER(vp)]),
    "zant_hip_conv2d_f32_packed": (i32, [vp, vp, vp, vp]),
    "zant_hip_conv2d_plan_destroy": (None, [vp, vp]),
    "zant_hip_conv2d_out_shape": (i32, [c_i64p, c_i64p, c_i64p, i32, c_i64p, i32, c_i64p, i32, i64, C.c_char_p, c_i64p]),
    "zant_hip_matmul_f32": (i32, [vp, vp, c_i64p, i32, vp, c_i64p, i32, vp]),
    "zant_hip_matmul_check": (i32, [c_i64p, i32, c_i64p, i32]),
    "zant_hip_gemm_f32": (i32, [vp, vp, c_i64p, vp, c_i64p, vp, c_i64p, i32, f32, f32, i32, i32, vp, c_i64p, i32]),
    "zant_hip_gemm_check": (i32, [c_i64p, i32, c_i64p, i32, c_i64p, i32, i32, i32, i32, c_i64p]),
    "zant_hip_maxpool2d_f32": (i32, [vp, vp, c_i64p, vp, c_i64p, c_i64p, c_i64p, c_i64p, c_i64p, i32, i32]),
    "zant_hip_maxpool2d_u8": (i32, [vp, vp, c_i64p, vp, c_i64p, c_i64p, c_i64p, c_i64p, c_i64p, i32, i32]),
    "zant_hip_maxpool2d_out_shape": (i32, [c_i64p, c_i64p, c_i64p, c_i64p, c_i64p, i32, i32, c_i64p]),
    "zant_hip_avgpool2d_f32": (i32, [vp, vp, c_i64p, vp, c_i64p, c_i64p, c_i64p, c_i64p, i32]),
    "zant_hip_avgpool2d_out_shape": (i32, [c_i64p, c_i64p, c_i64p, c_i64p, i32, c_i64p]),
    "zant_hip_batchnorm_f32": (i32, [vp, vp, c_i64p, i32, vp, vp, vp, vp, f32, vp]),
    "zant_hip_relu_f32": (i32, [vp, vp, vp, i64]),
    "zant_hip_leaky_relu_f32": (i32, [vp, vp, f32, vp, i64]),
    "zant_hip_softmax_f32": (i32, [vp, vp, vp, i64, i64]),
    "zant_hip_sigmoid_f32": (i32, [vp, vp, vp, i64]),
    "zant_hip_reduce_mean_f32": (i32, [vp, vp, c_i64p, i32, c_i64p, i32, i32, i32, vp, c_i64p, C.POINTER(i32)]),
    "zant_hip_concatenate": (i32, [vp, C.POINTER(vp), C.POINTER(c_i64p), C.POINTER(i32), i32, i64, sz, vp, c_i64p,
                                   C.POINTER(i32)]),
    "zant_hip_resize_nearest": (i32, [vp, vp, c_i64p, i32, sz, C.POINTER(f32), c_i64p, i32, i32, vp, c_i64p]),
    "zant_hip_add_f32": (i32, [vp, vp, c_i64p, i32, vp, c_i64p, i32, vp, c_i64p, C.POINTER(i32)]),
    "zant_hip_add_bias_f32": (i32, [vp, vp, c_i64p, i32, vp, c_i64p, i32]),
    "zant_hip_reshape": (i32, [vp, vp, c_i64p, i32, sz, c_i64p, i32, vp, c_i64p]),
    "zant_hip_quantize_linear_f32_u8": (i32, [vp, vp, c_i64p, i32, vp, vp, i64, i32, vp]),
    "zant_hip_dequantize_linear_u8_f32": (i32, [vp, vp, c_i64p, i32, vp, vp, i64, i32, vp]),
    "zant_hip_quantize_linear_f32_i8": (i32, [vp, vp, c_i64p, i32, vp, vp, i64, i32, vp]),
    "zant_hip_dequantize_linear_i8_f32": (i32, [vp, vp, c_i64p, i32, vp, vp, i64, i32, vp]),
    "zant_hip_dequantize_linear_i32_f32": (i32, [vp, vp, c_i64p, i32, vp, vp, i64, i32, vp]),
    "zant_hip_qlinearconv_u8i8": (i32, [vp, vp, c_i64p, f32, u8, vp, c_i64p, vp, i64, vp, f32, u8, vp, vp, c_i64p,
                                        c_i64p, c_i64p, c_i64p, i64, i32, f32, f32, u8]),
    "zant_hip_blocked16_bytes": (sz, [c_i64p]),
    "zant_hip_to_blocked16_u8": (i32, [vp, vp, c_i64p, vp]),
    "zant_hip_from_blocked16_u8": (i32, [vp, vp, c_i64p, vp]),
    "zant_hip_qlinearconv_prepack": (i32, [vp, c_i64p, f32, u8, vp, c_i64p, vp, i64, vp, f32, u8, vp, c_i64p, c_i64p,
                                           c_i64p, c_i64p, i64, i32, f32, f32, u8, i32, i32, C.POINTER(vp)]),
    "zant_hip_qlinearconv_u8i8_packed": (i32, [vp, vp, vp, vp]),
    "zant_hip_qlinearconv_plan_destroy": (None, [vp, vp]),
    "zant_hip_qlinear_act_u8": (i32, [vp, vp, i64, f32, u8, i32, f32, f32, u8, vp]),
    "zant_hip_qlinear_add_u8": (i32, [vp, vp, f32, u8, vp, f32, u8, f32, u8, vp, i64]),
    "zant_hip_qlinear_global_avgpool_u8": (i32, [vp, vp, c_i64p, f32, u8, f32, u8, vp]),
    "zant_model_create": (i32, [vp, C.POINTER(vp)]),
    "zant_model_destroy": (None, [vp]),
    "zant_model_input": (i32, [vp, i32, c_i64p, i32, f32, i32]),
    "zant_model_conv": (i32, [vp, i32, vp, c_i64p, vp, c_i64p, i32, c_i64p, i32, c_i64p, i32, i64, C.c_char_p]),
    "zant_model_relu": (i32, [vp, i32]),
    "zant_model_leaky_relu": (i32, [vp, i32, f32]),
    "zant_model_maxpool": (i32, [vp, i32, c_i64p, c_i64p, c_i64p, c_i64p, i32, i32]),
    "zant_model_avgpool": (i32, [vp, i32, c_i64p, c_i64p, c_i64p, i32, i32]),
    "zant_model_batchnorm": (i32, [vp, i32, vp, vp, vp, vp, i64, f32]),
    "zant_model_reshape": (i32, [vp, i32, c_i64p, i32]),
    "zant_model_gemm": (i32, [vp, i32, vp, c_i64p, vp, c_i64p, i32, f32, f32, i32, i32]),
    "zant_model_matmul": (i32, [vp, i32, vp, c_i64p, i32]),
    "zant_model_add_const": (i32, [vp, i32, vp, c_i64p, i32]),
    "zant_model_add": (i32, [vp, i32, i32]),
    "zant_model_softmax": (i32, [vp, i32]),
    "zant_model_sigmoid": (i32, [vp, i32]),
    "zant_model_reduce_mean": (i32, [vp, i32, c_i64p, i32, i32]),
    "zant_model_concat": (i32, [vp, C.POINTER(i32), i32, i64]),
    "zant_model_resize_nearest": (i32, [vp, i32, C.POINTER(f32), c_i64p, i32, i32]),
    "zant_model_quantize": (i32, [vp, i32, f32, i32]),
    "zant_model_dequantize": (i32, [vp, i32]),
    "zant_model_qlinearconv": (i32, [vp, i32, vp, c_i64p, vp, i64, vp, f32, i32, c_i64p, c_i64p, c_i64p, i64]),
    "zant_model_qlinear_act": (i32, [vp, i32, i32, f32, f32, i32]),
    "zant_model_qlinear_add": (i32, [vp, i32, i32, f32, i32]),
    "zant_model_qlinear_global_avgpool": (i32, [vp, i32, f32, i32]),
    "zant_model_finalize": (i32, [vp]),
    "zant_model_output_dims": (i32, [vp, c_i64p, C.POINTER(i32), C.POINTER(i32)]),
    "zant_model_tensor_dims": (i32, [vp, i32, c_i64p, C.POINTER(i32), C.POINTER(i32)]),
    "zant_model_arena_bytes": (sz, [vp]),
    "zant_model_unfused_bytes": (sz, [vp]),
    "zant_model_num_launches": (i32, [vp]),
    "zant_model_run": (i32, [vp, vp, vp]),
    "zant_model_input_ptr": (vp, [vp]),
    "zant_model_output_ptr": (vp, [vp]),
    "zant_model_predict_host": (i32, [vp, vp, vp]),
    "zant_model_profile": (i32, [vp, C.POINTER(f32), C.POINTER(C.c_double), C.POINTER(C.c_double), i32]),
    "zant_model_launch_name": (C.c_char_p, [vp, i32]),
    "zant_model_launch_kernel": (C.c_char_p, [vp, i32]),
    "zant_model_read_tensor": (i32, [vp, i32, vp, sz]),
    "zant_model_bind_predict": (i32, [vp]),
    "predict": (None, [vp, C.POINTER(C.c_uint32), C.c_uint32, C.POINTER(vp)]),
    "predict_batched": (None, [vp, C.c_uint32, C.POINTER(vp)]),
}

for _name, (_res, _args) in PROTOTYPES.items():
    _fn = getattr(lib, _name)  # AttributeError here = the header and the library disagree
    _fn.restype = _res
    _fn.argtypes = _args


def status_name(code):
    return lib.zant_hip_status_name(code).decode()


class ZantError(Exception):
    """A non-zero status from the library; ``name`` is the Zig error name the reference would return."""

    def __init__(self, code, detail=""):
        self.code = code
        self.name = status_name(code)
        super().__init__(self.name + (": " + detail if detail else ""))


def dims(seq):
    """(pointer, length) of a host int64 array, (None, 0) for None (Zig null)."""
    if seq is None:
        return None, 0
    n = len(seq)
    return (C.c_int64 * max(n, 1))(*[int(v) for v in seq]), n


class Context:
    """One zant_ctx = one HIP stream.  ``stream`` is a raw hipStream_t (int) or None for a private stream."""

    def __init__(self, device=0, stream=None):
        h = vp()
        rc = lib.zant_hip_ctx_create(C.byref(h), device, vp(stream) if stream else None)
        if rc:
            raise ZantError(rc, "zant_hip_ctx_create: " + lib.zant_hip_last_error(None).decode())
        self.handle = h

    def check(self, rc):
        if rc:
            raise ZantError(rc, lib.zant_hip_last_error(self.handle).decode() if rc == -100 else "")

    def sync(self):
        self.check(lib.zant_hip_sync(self.handle))

    def timer_start(self):
        self.check(lib.zant_hip_timer_start(self.handle))

    def timer_stop(self):
        ms = f32()
        self.check(lib.zant_hip_timer_stop(self.handle, C.byref(ms)))
        return ms.value

    def kernel_timing(self, enable):
        self.check(lib.zant_hip_kernel_timing(self.handle, int(enable)))

    def kernel_ms(self):
        ms = f32()
        self.check(lib.zant_hip_kernel_ms(self.handle, C.byref(ms)))
        return ms.value

    def kernel_name(self):
        """Device function of the last operator's main kernel ("" where the launch site does not name it)."""
        return lib.zant_hip_kernel_name(self.handle).decode()

    def close(self):
        if self.handle:
            lib.zant_hip_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

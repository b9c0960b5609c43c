"""ctypes binding of libwebgpt_amd.so (declared in include/webgpt_amd.h).

There is no fallback: if the shared library is missing, or a call fails, an
exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# WEBGPT_AMD_LIB selects another build of the same library (e.g. a profiling build).
LIB_PATH = os.environ.get("WEBGPT_AMD_LIB") or os.path.join(_HERE, "libwebgpt_amd.so")


class WgptError(RuntimeError):
    """A C-ABI call returned non-zero; the message is wgpt_last_error()."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


class Params(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layer", "n_head", "n_embd", "n_ctx", "vocab_size",
                                         "weight_dtype", "max_prefill", "flags")]


FLAG_TAPS = 1
FLAG_TUNE_DELAYS = 2

_u64 = C.c_uint64
_sz = C.c_size_t
_int = C.c_int
_vp = C.c_void_p
_fp = C.POINTER(C.c_float)
_ip = C.POINTER(C.c_int32)

# name -> (argtypes, checked): checked functions return an int status.
_SIGNATURES = {
    "wgpt_init": ([_int], True),
    "wgpt_shutdown": ([], True),
    "wgpt_device_info": ([C.c_char_p, _sz, C.POINTER(_int), C.POINTER(_u64)], True),
    "wgpt_alloc": ([_sz, C.POINTER(_u64)], True),
    "wgpt_free": ([_u64], True),
    "wgpt_buf_size": ([_u64, C.POINTER(_sz)], True),
    "wgpt_upload": ([_u64, _sz, _vp, _sz], True),
    "wgpt_download": ([_vp, _u64, _sz, _sz], True),
    "wgpt_copy": ([_u64, _sz, _u64, _sz, _sz], True),
    "wgpt_sync": ([], True),
    "wgpt_matmul_bias": ([_int, _int, _int, _u64, _u64, _u64, _u64], True),
    "wgpt_matmul_bias_noalloc": ([_int, _int, _int, _u64, _u64, _u64, _u64], True),
    "wgpt_matmul_bias_i8": ([_int, _int, _int, _u64, _u64, _u64, _u64, _u64], True),
    "wgpt_dequant_i8": ([_int, _int, _u64, _u64, _u64], True),
    "wgpt_residual": ([_int, _int, _u64, _u64, _u64], True),
    "wgpt_layernorm": ([_int, _int, _u64, _u64, _u64, _u64], True),
    "wgpt_softmax": ([_int, _int, _u64, _u64], True),
    "wgpt_softmax_t": ([_int, _int, _u64, _u64], True),
    "wgpt_transpose": ([_int, _int, _u64, _u64], True),
    "wgpt_gelu": ([_int, _int, _u64, _u64], True),
    "wgpt_embed": ([_ip, _int, _int, _int, _u64, _u64, _u64], True),
    "wgpt_deembed": ([_int, _int, _int, _u64, _u64, _u64], True),
    "wgpt_attention": ([_int, _int, C.c_float, _int, _int] + [_u64] * 10, True),
    "wgpt_sample_topk": ([_int, _int, C.c_double, C.c_double, _u64, _ip, _ip, C.POINTER(C.c_double)], True),
    "wgpt_model_create": ([C.POINTER(Params), C.POINTER(_u64)], True),
    "wgpt_model_set_tensor": ([_u64, C.c_char_p, _vp, _sz], True),
    "wgpt_model_finalize": ([_u64], True),
    "wgpt_prefill": ([_u64, _ip, _int, _fp], True),
    "wgpt_decode": ([_u64, C.c_int32, _fp], True),
    "wgpt_decode_greedy": ([_u64, C.c_int32, _int, _ip, _fp], True),
    "wgpt_decode_sample": ([_u64, C.c_int32, _int, _int, C.c_double, C.POINTER(C.c_double), _ip, _fp], True),
    "wgpt_model_reset_cache": ([_u64], True),
    "wgpt_model_position": ([_u64, C.POINTER(_int)], True),
    "wgpt_model_tap": ([_u64, C.c_char_p, _fp, _sz], True),
    "wgpt_model_last_gpu_ms": ([_u64, _fp], True),
    "wgpt_model_decode_bytes": ([_u64, _int, C.POINTER(_u64)], True),
    "wgpt_model_set_decode_mode": ([_u64, _int], True),
    "wgpt_model_tune_poll_delays": ([_u64, _int, _ip, _fp, _fp], True),
    "wgpt_model_poll_delays": ([_u64, _ip], True),
    "wgpt_model_destroy": ([_u64], True),
    "wgpt_synth_normal": ([C.c_uint32, C.c_uint32, _sz, C.c_double, _fp], False),
    "wgpt_synth_tokens": ([C.c_uint32, C.c_uint32, _sz, C.c_uint32, _ip], False),
    "wgpt_synth_int8_packed": ([C.c_uint32, C.c_uint32, _sz, _sz, _ip], False),
    "wgpt_synth_uniform": ([C.c_uint32, C.c_uint32, _sz, C.c_double, C.c_double, _fp], False),
}

EXPORTS = sorted(list(_SIGNATURES) + ["wgpt_last_error", "wgpt_synth_tensor_id"])

_cdll = None


def cdll():
    """The loaded shared library (raises if it has not been built)."""
    global _cdll
    if _cdll is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C webgpt_amd/csrc` "
                "(or __graft_entry__.build()); there is no fallback implementation")
        lib = C.CDLL(LIB_PATH)
        lib.wgpt_last_error.restype = C.c_char_p
        lib.wgpt_last_error.argtypes = []
        lib.wgpt_synth_tensor_id.restype = C.c_uint32
        lib.wgpt_synth_tensor_id.argtypes = [C.c_char_p]
        for name, (argtypes, checked) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _int if checked else None
        _cdll = lib
    return _cdll


def call(name, *args):
    """Calls a status-returning entry point; raises WgptError on failure."""
    lib = cdll()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise WgptError(rc, lib.wgpt_last_error().decode("utf-8", "replace"))


_initialised = False


def init(device=0):
    global _initialised
    call("wgpt_init", device)
    _initialised = True


def shutdown():
    global _initialised
    call("wgpt_shutdown")
    _initialised = False

"""ctypes binding of libcaten_hip.so (the C ABI declared in include/caten_hip.h).

There is no CPU fallback: if the library is missing or a call fails the error is
raised, the way Caten's CLANG backend raises when gcc fails
(source/byoc/clang.lisp:150-156).
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcaten_hip.so")

# constants of include/caten_hip.h
F32, F16, Q4_0, Q8_0 = 0, 1, 2, 8
GGML_TYPE = {"f32": F32, "f16": F16, "q4_0": Q4_0, "q8_0": Q8_0}
PRO_NONE, PRO_LAYERNORM, PRO_RMSNORM, PRO_SWIGLU = 0, 1, 2, 3
ACT_NONE, ACT_RELU, ACT_GELU, ACT_SILU, ACT_SIGMOID, ACT_TANH = 0, 1, 2, 3, 4, 5
ARCH_GPT2, ARCH_LLAMA = 0, 1


class HipError(RuntimeError):
    """A non-zero status from libcaten_hip.so (message from cthip_last_error)."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[cthip {code}] {message}")
        self.code = code


class DecoderConfig(C.Structure):
    _fields_ = [("arch", C.c_int), ("n_layers", C.c_int), ("dim", C.c_int), ("n_heads", C.c_int),
                ("n_kv_heads", C.c_int), ("ffn", C.c_int), ("vocab", C.c_int), ("max_seq", C.c_int),
                ("eps", C.c_float), ("rope_base", C.c_float)]


_vp, _vpp = C.c_void_p, C.POINTER(C.c_void_p)
_i, _i64, _sz, _f = C.c_int, C.c_int64, C.c_size_t, C.c_float

# name -> (restype, argtypes); every symbol include/caten_hip.h declares
PROTOTYPES = {
    "cthip_init": (_i, [_i]),
    "cthip_shutdown": (_i, []),
    "cthip_last_error": (C.c_char_p, []),
    "cthip_device_info": (_i, [C.c_char_p, _i, C.POINTER(_i), C.POINTER(_i), C.POINTER(_sz), C.POINTER(_sz)]),
    "cthip_alloc": (_i, [_vpp, _sz]),
    "cthip_free": (_i, [_vp]),
    "cthip_cache_trim": (_i, []),
    "cthip_cache_stats": (_i, [C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz)]),
    "cthip_h2d": (_i, [_vp, _vp, _sz]),
    "cthip_d2h": (_i, [_vp, _vp, _sz]),
    "cthip_d2d": (_i, [_vp, _vp, _sz]),
    "cthip_memset": (_i, [_vp, _i, _sz]),
    "cthip_sync": (_i, []),
    "cthip_stream": (_vp, []),
    "cthip_compile": (_i, [C.c_char_p, C.c_char_p, _vpp, C.POINTER(_sz), C.POINTER(C.c_void_p)]),
    "cthip_release": (None, [_vp]),
    "cthip_module_load": (_i, [_vpp, _vp]),
    "cthip_module_unload": (_i, [_vp]),
    "cthip_get_function": (_i, [_vpp, _vp, C.c_char_p]),
    "cthip_launch": (_i, [_vp, C.POINTER(C.c_uint), C.POINTER(C.c_uint), C.c_uint, _vpp, _i]),
    "cthip_render_header": (C.c_char_p, []),
    "cthip_program_create": (_i, [_vpp, C.c_char_p]),
    "cthip_program_destroy": (_i, [_vp]),
    "cthip_program_source": (C.c_char_p, [_vp]),
    "cthip_program_name": (C.c_char_p, [_vp]),
    "cthip_program_route": (C.c_char_p, [_vp]),
    "cthip_program_last_route": (C.c_char_p, [_vp]),
    "cthip_program_bind": (_i, [_vp, _vp]),
    "cthip_program_launch": (_i, [_vp, C.POINTER(C.c_void_p), _i]),
    "cthip_vm_create": (_i, [_vpp, _i]),
    "cthip_vm_destroy": (_i, [_vp]),
    "cthip_vm_add_scalar": (_i, [_vp, _i, _i, _i, C.POINTER(_i), C.POINTER(C.c_longlong), C.POINTER(C.c_double)]),
    "cthip_vm_add_allocate": (_i, [_vp, _i, _i, _i, C.POINTER(_i), C.POINTER(C.c_longlong)]),
    "cthip_vm_add_kernel": (_i, [_vp, _vp, _i, C.POINTER(_i), C.POINTER(C.c_longlong), C.POINTER(C.c_double), C.POINTER(_i),
                                 _i, C.POINTER(_i), C.POINTER(_i)]),
    "cthip_vm_set_int": (_i, [_vp, _i, C.c_longlong]),
    "cthip_vm_set_float": (_i, [_vp, _i, C.c_double]),
    "cthip_vm_set_buffer": (_i, [_vp, _i, _vp]),
    "cthip_vm_run": (_i, [_vp]),
    "cthip_vm_get": (_i, [_vp, _i, C.POINTER(_i), C.POINTER(C.c_longlong), C.POINTER(C.c_double), _vpp]),
    "cthip_vm_launches": (C.c_longlong, [_vp]),
    "cthip_timer_start": (_i, []),
    "cthip_timer_stop": (_i, [C.POINTER(_f)]),
    "cthip_dequant": (_i, [_i, _vp, _i64, _vp]),
    "cthip_wmat_create": (_i, [_vpp, _i, _vp, _i64, _i64]),
    "cthip_wmat_destroy": (_i, [_vp]),
    "cthip_wmat_nbytes": (_i64, [_vp]),
    "cthip_wmat_dequant": (_i, [_vp, _vp]),
    "cthip_wmat_fold_layernorm": (_i, [_vp, _vp, _vp, _vp]),
    "cthip_linear": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _i, _i, _vp, _vp, _f]),
    "cthip_set_option": (_i, [C.c_char_p, _i]),
    "cthip_matmul": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "cthip_matmul_noalloc": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "cthip_softmax": (_i, [_vp, _vp, _i64, _i]),
    "cthip_layernorm": (_i, [_vp, _vp, _vp, _vp, _f, _i64, _i]),
    "cthip_rmsnorm": (_i, [_vp, _vp, _vp, _f, _i64, _i]),
    "cthip_layernorm_softmax": (_i, [_vp, _vp, _vp, _vp, _f, _i64, _i]),
    "cthip_unary": (_i, [_i, _vp, _vp, _i64]),
    "cthip_embedding": (_i, [_vp, _vp, _vp, _i, _i, _i]),
    "cthip_argmax": (_i, [_vp, _vp, _i64, _i]),
    "cthip_rope": (_i, [_vp, _vp, _i, _i, _i, _i, _f, _i]),
    "cthip_sdpa_cached": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "cthip_kv_append_q8": (_i, [_vp, _vp, _vp, _i, _i, _i]),
    "cthip_sdpa_cached_q8": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    "cthip_kv_page_rows": (_i, []),
    "cthip_kv_append_paged": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "cthip_sdpa_cached_paged": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    "cthip_decoder_create": (_i, [_vpp, C.POINTER(DecoderConfig)]),
    "cthip_decoder_destroy": (_i, [_vp]),
    "cthip_decoder_load": (_i, [_vp, C.c_char_p, _i, _vp, _i64, _i64]),
    "cthip_decoder_missing": (_i, [_vp]),
    "cthip_decoder_forward": (_i, [_vp, _vp, _i, _i, C.POINTER(_i64), _vp]),
    "cthip_decoder_generate": (_i, [_vp, _i, _vp]),
    "cthip_decoder_generate_until": (_i, [_vp, _i, _i64, _vp, C.POINTER(_i)]),
    "cthip_decoder_position": (_i, [_vp]),
    "cthip_decoder_step_bytes": (_i64, [_vp, _i]),
    "cthip_decoder_layer_launches": (_i, [_vp]),
    "cthip_decoder_peek": (_i, [_vp, C.c_char_p, _vpp, C.POINTER(_i64)]),
    "cthip_gguf_open": (_i, [_vpp, C.c_char_p]),
    "cthip_gguf_close": (_i, [_vp]),
    "cthip_gguf_version": (_i, [_vp]),
    "cthip_gguf_tensor_count": (_i64, [_vp]),
    "cthip_gguf_metadata_count": (_i64, [_vp]),
    "cthip_gguf_alignment": (_i64, [_vp]),
    "cthip_gguf_tensor_info": (_i, [_vp, _i64, C.POINTER(C.c_char_p), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i64),
                                    C.POINTER(_i64), C.POINTER(_i64)]),
    "cthip_gguf_find_tensor": (_i64, [_vp, C.c_char_p]),
    "cthip_gguf_tensor_data": (_vp, [_vp, _i64]),
    "cthip_gguf_find_metadata": (_i64, [_vp, C.c_char_p]),
    "cthip_gguf_metadata_info": (_i, [_vp, _i64, C.POINTER(C.c_char_p), C.POINTER(_i), C.POINTER(_i), C.POINTER(_i64)]),
    "cthip_gguf_metadata_number": (_i, [_vp, _i64, C.POINTER(C.c_double)]),
    "cthip_gguf_metadata_string": (_i, [_vp, _i64, _i64, C.POINTER(C.c_void_p), C.POINTER(_i64)]),
    "cthip_decoder_load_gguf": (_i, [_vp, _vp, _i, C.POINTER(_i)]),
    "cthip_bpe_create": (_i, [_vpp, C.c_char_p, _sz, C.c_char_p, _sz]),
    "cthip_bpe_destroy": (_i, [_vp]),
    "cthip_bpe_vocab_size": (_i, [_vp]),
    "cthip_bpe_encode": (_i, [_vp, C.c_char_p, _sz, C.POINTER(_i), _sz, C.POINTER(_sz)]),
    "cthip_bpe_decode": (_i, [_vp, C.POINTER(_i), _sz, C.c_char_p, _sz, C.POINTER(_sz)]),
}

E_NOT_INIT, E_BAD_ARG, E_UNSUPPORTED, E_COMPILE, E_STATE = -1, -2, -3, -4, -5  # include/caten_hip.h

_lib = None
_inited = False


def load() -> C.CDLL:
    """dlopen the library and type every entry point.  Needs no GPU."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipError(-1, f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                               "(make -C caten_amd/csrc)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)  # AttributeError here = the header and the library disagree
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status: int) -> None:
    if status != 0:
        msg = load().cthip_last_error()
        raise HipError(status, msg.decode("utf-8", "replace") if msg else "unknown error")


def init(device: int = 0) -> C.CDLL:
    """cthip_init; raises if there is no gfx950 device."""
    global _inited
    lib = load()
    if not _inited:
        check(lib.cthip_init(device))
        _inited = True
    return lib


def is_initialised() -> bool:
    return _inited

"""ctypes binding of libhq.so (the C-ABI declared in include/hq.h).

The library is built in-tree by ``hecbench_amd.build`` (hipcc, gfx950) and is
the only compute path: if it is missing, importing this module raises, there is
no CPU or PyTorch fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhq.so")

# Every symbol include/hq.h declares, with its ctypes signature.
_c = ctypes
_SIGNATURES = {
    "hq_abi_version": (_c.c_int, []),
    "hq_strerror": (_c.c_char_p, [_c.c_int]),
    "hq_init": (_c.c_int, []),
    "hq_reserve_workspace": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_int]),
    "hq_q3_workspace_need": (_c.c_int, [_c.c_int, _c.c_int, _c.c_int, _c.c_int, _c.POINTER(_c.c_int64),
                                        _c.POINTER(_c.c_int64)]),
    "hq_reserve_need": (_c.c_int, [_c.c_int, _c.c_int, _c.c_int, _c.POINTER(_c.c_int64), _c.POINTER(_c.c_int64)]),
    "hq_shutdown": (_c.c_int, []),
    "hq_set_tunable": (_c.c_int, [_c.c_char_p, _c.c_int, _c.c_int]),
    "hq_device_info": (_c.c_int, [_c.POINTER(_c.c_int)] * 5 + [_c.c_char_p, _c.c_int]),
    "hq_dequant_nf4": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int,
                                  _c.c_int, _c.c_void_p]),
    "hq_quantize_dynamic8": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64,
                                        _c.c_void_p]),
    "hq_q3_matvec": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_void_p,
                                _c.c_void_p, _c.c_int, _c.c_int, _c.c_int, _c.c_uint, _c.c_void_p]),
    "hq_q3_matvec_noalloc": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_void_p,
                                        _c.c_void_p, _c.c_int, _c.c_int, _c.c_int, _c.c_uint, _c.c_void_p]),
    "hq_lut_gemv": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
                               _c.c_int, _c.c_int, _c.c_int, _c.c_int, _c.c_void_p]),
    "hq_q3_matvec_plan": (_c.c_int, [_c.c_int, _c.c_int, _c.c_int]),
    "hq_lut_gemv_plan": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int, _c.c_int, _c.c_int]),
    "hq_aqlm_matvec": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p,
                                  _c.c_int, _c.c_int, _c.POINTER(_c.c_int), _c.c_int, _c.c_void_p]),
    "hq_q3_pack": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int, _c.c_void_p]),
    "hq_bcq_pack": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int, _c.c_int, _c.c_void_p]),
    "hq_quantize_4bit": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int,
                                    _c.c_int, _c.c_void_p]),
    "hq_int8_quant_static": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int64, _c.c_int, _c.c_float,
                                        _c.c_int, _c.c_int32, _c.c_void_p]),
    "hq_int8_quant_dynamic": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64,
                                         _c.c_int, _c.c_void_p]),
    "hq_gemv_fp16": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int, _c.c_void_p]),
    "hq_gemv_int8": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int, _c.c_float,
                                _c.c_float, _c.c_void_p]),
    "hq_gemv_int4": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int, _c.c_float,
                                _c.c_float, _c.c_void_p]),
    "hq_mxfp4_qdq": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int, _c.c_void_p]),
    "hq_probe_stream": (_c.c_int, [_c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_void_p]),
    "hq_probe_gather16": (_c.c_int, [_c.c_void_p, _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_void_p]),
    "hq_probe_gather16_count": (_c.c_int64, [_c.c_int64]),
    "hq_probe_lds": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_int, _c.c_int, _c.c_void_p, _c.c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


def load():
    """Load libhq.so once and attach the signatures.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `python -m hecbench_amd.build` (needs hipcc)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class HqError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        msg = load().hq_strerror(code).decode()
        super().__init__(f"{where}: {msg} (code {code})")


def check(code, where):
    if code != 0:
        raise HqError(code, where)

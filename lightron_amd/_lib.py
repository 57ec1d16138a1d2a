"""ctypes binding of include/ltr_attn.h.  No fallback: if the shared library is missing the
import of any compute entry point raises, and a GPU call on a non-gfx950 device returns
LTR_EDEVICE from the library."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# LTR_ATTN_LIB names another build of the same library (same ABI version), e.g. to compare two builds in one session
LIB_PATH = os.environ.get("LTR_ATTN_LIB") or os.path.join(HERE, "csrc", "libltr_attn.so")

LTR_ABI_VERSION = 8
LTR_MAX_CHUNKS = 32
LTR_NOALLOC_MAX_ROWS = 1 << 20
LTR_BF16, LTR_F32 = 0, 1
LTR_CAUSAL, LTR_MERGE, LTR_NO_DQ, LTR_NO_DKDV, LTR_DQ_BF16, LTR_DELTA_FROM_O, LTR_DKDV_BF16 = 1, 2, 4, 8, 16, 32, 64
LTR_ROPE_Q, LTR_ROPE_DQ = 128, 256
LTR_DKDV_KEYS_128, LTR_DKDV_KEYS_256 = 512, 1024
LTR_DQ_ROWS_256, LTR_DQ_ROWS_512 = 2048, 4096
LTR_FWD_ROWS_256, LTR_FWD_ROWS_512 = 8192, 16384
LTR_FWD_F32_SCALAR = 32768
LTR_BWD_F32_SCALAR = 65536

EXPORTS = ("ltr_attn_fwd", "ltr_attn_bwd_delta", "ltr_attn_bwd", "ltr_attn_bwd_noalloc", "ltr_attn_plan", "ltr_cast_f32_to_bf16",
           "ltr_rope_apply", "ltr_abi_version", "ltr_strerror")
# the bench-only measurement library (include/ltr_probe.h); not part of the attention path
PROBE_LIB_PATH = os.path.join(HERE, "csrc", "libltr_probe.so")
PROBE_EXPORTS = ("ltr_device_info", "ltr_probe_mfma")

_i64x3 = ctypes.c_int64 * 3
_i64x2 = ctypes.c_int64 * 2


class KvChunk(ctypes.Structure):
    _fields_ = [("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("dk", ctypes.c_void_p), ("dv", ctypes.c_void_p),
                ("sk", ctypes.c_int64), ("pos0", ctypes.c_int64)]


class FwdArgs(ctypes.Structure):
    _fields_ = [("q", ctypes.c_void_p), ("o", ctypes.c_void_p), ("lse", ctypes.c_void_p),
                ("B", ctypes.c_int32), ("Hq", ctypes.c_int32), ("Hkv", ctypes.c_int32), ("D", ctypes.c_int32),
                ("Sq", ctypes.c_int64),
                ("q_stride", _i64x3), ("o_stride", _i64x3), ("k_stride", _i64x3), ("v_stride", _i64x3),
                ("q_pos0", _i64x2), ("q_split", ctypes.c_int64),
                ("scale", ctypes.c_float), ("flags", ctypes.c_uint32),
                ("io_dtype", ctypes.c_int32), ("o_dtype", ctypes.c_int32), ("n_chunks", ctypes.c_int32),
                ("chunk", KvChunk * LTR_MAX_CHUNKS),
                ("rope_freqs", ctypes.c_void_p), ("rope_pos0", ctypes.c_int64), ("rope_len", ctypes.c_int64),
                ("q_rot", ctypes.c_void_p), ("q_rot_stride", _i64x3)]


class DeltaArgs(ctypes.Structure):
    _fields_ = [("o", ctypes.c_void_p), ("d_o", ctypes.c_void_p), ("delta", ctypes.c_void_p),
                ("B", ctypes.c_int32), ("Hq", ctypes.c_int32), ("D", ctypes.c_int32),
                ("Sq", ctypes.c_int64),
                ("o_stride", _i64x3), ("do_stride", _i64x3),
                ("o_dtype", ctypes.c_int32), ("do_dtype", ctypes.c_int32)]


class BwdArgs(ctypes.Structure):
    _fields_ = [("q", ctypes.c_void_p), ("d_o", ctypes.c_void_p), ("lse", ctypes.c_void_p),
                ("delta", ctypes.c_void_p), ("dq", ctypes.c_void_p),
                ("B", ctypes.c_int32), ("Hq", ctypes.c_int32), ("Hkv", ctypes.c_int32), ("D", ctypes.c_int32),
                ("Sq", ctypes.c_int64),
                ("q_stride", _i64x3), ("do_stride", _i64x3), ("dq_stride", _i64x3),
                ("k_stride", _i64x3), ("v_stride", _i64x3), ("dk_stride", _i64x3), ("dv_stride", _i64x3),
                ("q_pos0", _i64x2), ("q_split", ctypes.c_int64),
                ("scale", ctypes.c_float), ("flags", ctypes.c_uint32),
                ("io_dtype", ctypes.c_int32), ("n_chunks", ctypes.c_int32),
                ("chunk", KvChunk * LTR_MAX_CHUNKS),
                ("o", ctypes.c_void_p), ("o_stride", _i64x3),
                ("rope_freqs", ctypes.c_void_p), ("rope_pos0", ctypes.c_int64), ("rope_len", ctypes.c_int64)]


class RopeArgs(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("out", ctypes.c_void_p), ("freqs", ctypes.c_void_p),
                ("B", ctypes.c_int32), ("H", ctypes.c_int32), ("D", ctypes.c_int32),
                ("S", ctypes.c_int64),
                ("x_stride", _i64x3), ("out_stride", _i64x3),
                ("flags", ctypes.c_uint32), ("io_dtype", ctypes.c_int32)]


class DeviceInfo(ctypes.Structure):
    _fields_ = [("compute_units", ctypes.c_int32), ("clock_khz", ctypes.c_int32), ("memory_clock_khz", ctypes.c_int32),
                ("memory_bus_bits", ctypes.c_int32), ("lds_bytes_per_block", ctypes.c_int64), ("hbm_bytes", ctypes.c_int64),
                ("arch", ctypes.c_char * 64)]


class AttnPlan(ctypes.Structure):
    _fields_ = [("compute_units", ctypes.c_int32), ("fwd_rows", ctypes.c_int32), ("fwd_paired", ctypes.c_int32),
                ("dq_rows", ctypes.c_int32), ("dq_paired", ctypes.c_int32), ("dkdv_keys", ctypes.c_int32),
                ("fwd_blocks", ctypes.c_int64), ("dq_blocks", ctypes.c_int64), ("dkdv_blocks", ctypes.c_int64),
                ("fwd_kernel", ctypes.c_char * 48), ("dq_kernel", ctypes.c_char * 48), ("dkdv_kernel", ctypes.c_char * 48)]


LTR_PROBE_MIN_WORKSPACE = 8192 + 65536

_lib = None
_probe = None


def load():
    """Load (once) and return the ctypes handle; raises if the extension has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "lightron_amd: %s is missing - build it with `python -m lightron_amd.build` "
            "(there is no CPU or PyTorch fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    lib.ltr_attn_fwd.argtypes = [ctypes.POINTER(FwdArgs), ctypes.c_void_p]
    lib.ltr_attn_fwd.restype = ctypes.c_int
    lib.ltr_attn_bwd_delta.argtypes = [ctypes.POINTER(DeltaArgs), ctypes.c_void_p]
    lib.ltr_attn_bwd_delta.restype = ctypes.c_int
    lib.ltr_attn_bwd.argtypes = [ctypes.POINTER(BwdArgs), ctypes.c_void_p]
    lib.ltr_attn_bwd.restype = ctypes.c_int
    lib.ltr_attn_bwd_noalloc.argtypes = [ctypes.POINTER(BwdArgs), ctypes.c_void_p]
    lib.ltr_attn_bwd_noalloc.restype = ctypes.c_int
    lib.ltr_cast_f32_to_bf16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    lib.ltr_cast_f32_to_bf16.restype = ctypes.c_int
    lib.ltr_rope_apply.argtypes = [ctypes.POINTER(RopeArgs), ctypes.c_void_p]
    lib.ltr_rope_apply.restype = ctypes.c_int
    lib.ltr_attn_plan.argtypes = [ctypes.POINTER(BwdArgs), ctypes.POINTER(AttnPlan)]
    lib.ltr_attn_plan.restype = ctypes.c_int
    lib.ltr_abi_version.argtypes = []
    lib.ltr_abi_version.restype = ctypes.c_int
    lib.ltr_strerror.argtypes = [ctypes.c_int]
    lib.ltr_strerror.restype = ctypes.c_char_p
    if lib.ltr_abi_version() != LTR_ABI_VERSION:
        raise RuntimeError("lightron_amd: ABI version mismatch (library %d, binding %d)"
                           % (lib.ltr_abi_version(), LTR_ABI_VERSION))
    _lib = lib
    return lib


def load_probe():
    """The measurement library of bench.py (device facts, matrix-pipe ceiling probe); raises if it has not been built."""
    global _probe
    if _probe is not None:
        return _probe
    if not os.path.exists(PROBE_LIB_PATH):
        raise RuntimeError("lightron_amd: %s is missing - build it with `python -m lightron_amd.build`" % PROBE_LIB_PATH)
    lib = ctypes.CDLL(PROBE_LIB_PATH)
    lib.ltr_device_info.argtypes = [ctypes.POINTER(DeviceInfo)]
    lib.ltr_device_info.restype = ctypes.c_int
    lib.ltr_probe_mfma.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
    lib.ltr_probe_mfma.restype = ctypes.c_int
    _probe = lib
    return lib


def check(rc: int, what: str):
    if rc != 0:
        raise RuntimeError("%s failed: %s (%d)" % (what, load().ltr_strerror(rc).decode(), rc))

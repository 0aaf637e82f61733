"""ctypes binding of libhbstep.so (the C ABI declared in include/hbstep.h).

The library is built in-tree by ``make -C heavyball_amd/csrc`` (or ``__graft_entry__.build()``).  There is no
fallback: if the shared object is missing, or a call returns an error, this module raises.
"""

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int32, c_int64, c_uint32, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
# HBSTEP_LIB names another build of the library (same ABI), e.g. one compiled with different tuning constants
LIB_PATH = os.environ.get("HBSTEP_LIB") or os.path.join(_HERE, "libhbstep.so")

# include/hbstep.h
ABI_VERSION = 12  # HB_ABI_VERSION this binding was written against
FMT_F32, FMT_BF16, FMT_F16, FMT_ECC_BF16_8, FMT_ECC_BF16_16, FMT_ECC_F16_8, FMT_ECC_F16_16 = range(7)
ALGO_ADAM, ALGO_LAPROP, ALGO_ADOPT, ALGO_ADEMAMIX, ALGO_NADAM = range(5)
FLAG_MARS, FLAG_CAUTION, FLAG_CAUTIOUS_WD, FLAG_WRITE_GRAD, FLAG_UPDATE_ONLY, FLAG_ADOPT_WARMUP, FLAG_COUPLED_WD, FLAG_MARS_ONLY = 1, 2, 4, 8, 16, 32, 64, 128
RNG_HALF, RNG_PHILOX = 0, 1
STREAM_MARS_SR, STREAM_PARAM, STREAM_EXP_AVG, STREAM_EXP_AVG_SQ, STREAM_OLD_GRAD, STREAM_INIT_PARAM, STREAM_NS_INPUT = range(7)
STREAM_CLIP, STREAM_EXP_AVG_SLOW, STREAM_UPDATE, STREAM_SOAP_ROTATE, STREAM_UPDATE_CLIP = 8, 9, 10, 11, 12
STREAM_SOAP_GG, STREAM_SOAP_Q = 16, 17  # + 2 * side
NS_LEGACY, NS_BF16_UPDATE, NS_F16_UPDATE, NS_APPLY_TO_PARAM, NS_CAUTIOUS_WD = 1, 2, 4, 8, 16
NOALLOC_MAX_TENSORS = 8192  # HB_NOALLOC_MAX_TENSORS
CAUTION_SLOTS = 32  # HB_CAUTION_SLOTS: counters per tensor in HbStepDesc.caution_count
GEMM_ACCUMULATE, GEMM_SYMMETRIC = 1, 2
ORTHO_MAX_BATCH = 64  # HB_ORTHO_MAX_BATCH: matrices per hb_orthonormalize_f32_batched call
MOM_NESTEROV_EMA, MOM_EMA, MOM_HEAVYBALL, MOM_NESTEROV_HEAVYBALL = range(4)

ECC_FMT = {"bf16+8": FMT_ECC_BF16_8, "bf16+16": FMT_ECC_BF16_16, "fp16+8": FMT_ECC_F16_8, "fp16+16": FMT_ECC_F16_16}


class HbStepDesc(Structure):
    _fields_ = [
        ("param", c_void_p),
        ("param_corr", c_void_p),
        ("grad", c_void_p),
        ("grad_ptrs", c_void_p),
        ("exp_avg", c_void_p),
        ("exp_avg_corr", c_void_p),
        ("exp_avg_sq", c_void_p),
        ("exp_avg_sq_corr", c_void_p),
        ("old_grad", c_void_p),
        ("old_grad_corr", c_void_p),
        ("offsets", c_void_p),
        ("numel", c_void_p),
        ("chunks", c_void_p),
        ("caution_count", c_void_p),
        ("n_chunks", c_int64),
        ("n_tensors", c_int32),
        ("algo", c_int32),
        ("flags", c_uint32),
        ("param_fmt", c_int32),
        ("grad_fmt", c_int32),
        ("state_fmt", c_int32),
        ("a1", c_float),
        ("one_minus_a1", c_float),
        ("a2", c_float),
        ("one_minus_a2", c_float),
        ("mars_a", c_float),
        ("one_minus_mars_a", c_float),
        ("neg_lr", c_float),
        ("one_minus_decay_lr", c_float),
        ("eps", c_float),
        ("rng_mode", c_int32),
        ("step", c_uint32),
        ("seed", c_uint64),
        ("exp_avg_slow", c_void_p),
        ("exp_avg_slow_corr", c_void_p),
        ("a3", c_float),
        ("one_minus_a3", c_float),
        ("alpha", c_float),
        ("coupled_wd", c_float),
        ("tensor_scalars", c_void_p),
        ("update_out", c_void_p),
    ]


_PROTOTYPES = {
    "hb_fused_step": (ctypes.c_int, [POINTER(HbStepDesc), c_void_p]),
    "hb_fused_step_noalloc": (ctypes.c_int, [POINTER(HbStepDesc), c_void_p]),
    "hb_update_param": (ctypes.c_int, [POINTER(HbStepDesc), c_void_p]),
    "hb_ecc_encode": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_uint64, c_uint32, c_uint32, c_int64, c_void_p]),
    "hb_ecc_decode": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_void_p]),
    "hb_sr_bf16": (ctypes.c_int, [c_void_p, c_void_p, c_int64, c_int32, c_uint64, c_uint32, c_uint32, c_int64, c_void_p]),
    "hb_philox_words": (ctypes.c_int, [c_void_p, c_int64, c_uint64, c_uint64, c_uint32, c_uint32, c_void_p]),
    "hb_sumsq": (ctypes.c_int, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p]),
    "hb_scale": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "hb_nesterov_ema": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_float, c_float, c_void_p]),
    "hb_momentum": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
                                   c_int32, c_float, c_float, c_int32, c_uint64, c_uint32, c_void_p]),
    "hb_momentum_sumsq": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
                                         c_int32, c_float, c_float, c_int32, c_uint64, c_uint32, c_void_p, c_void_p]),
    "hb_momentum_sumsq_parts_per_chunk": (ctypes.c_int, []),
    "hb_ns5_workspace_bytes": (ctypes.c_int, [c_int64, c_int64, POINTER(c_int64)]),
    "hb_ns5_batched_workspace_bytes": (ctypes.c_int, [c_int32, POINTER(c_int64), POINTER(c_int64), POINTER(c_int64)]),
    "hb_ns5_batched": (ctypes.c_int, [c_int32, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64), POINTER(c_int64), POINTER(c_float),
                                      c_int32, c_float, POINTER(c_float), c_int32, c_uint64, c_uint32, POINTER(c_int64), c_void_p, c_int64,
                                      c_void_p]),
    "hb_ns5_batched_mixed": (ctypes.c_int, [c_int32, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64), POINTER(c_int64), POINTER(c_float),
                                            POINTER(c_int32), c_float, POINTER(c_float), c_int32, c_uint64, c_uint32, POINTER(c_int64), c_void_p,
                                            c_int64, c_void_p]),
    "hb_ns_batched_steps": (ctypes.c_int, [c_int32, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64), POINTER(c_int64), c_int32, POINTER(c_float),
                                           POINTER(c_int32), c_float, POINTER(c_float), POINTER(c_float), POINTER(c_void_p), POINTER(c_int32),
                                           c_int32, c_uint64, c_uint32, POINTER(c_int64), c_void_p, c_int64, c_void_p]),
    "hb_ns_tile": (ctypes.c_int, [c_int64, c_int64]),
    "hb_ns_product": (ctypes.c_int, [c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_float, c_float, c_void_p,
                                     c_int64, c_void_p]),
    "hb_ns5": (ctypes.c_int, [c_void_p, c_void_p, c_int64, c_int64, POINTER(c_float), c_int32, c_float, c_float, c_int32, c_uint64, c_uint32,
                              c_int64, c_void_p, c_int64, c_void_p]),
    "hb_gemm_f32": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int32, c_int32, c_int32,
                                   c_float, c_float, c_void_p]),
    "hb_gemm_f32_grouped": (ctypes.c_int, [c_int32, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64), POINTER(c_int64),
                                           POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), POINTER(c_int64), c_int32, c_int32, POINTER(c_int32),
                                           POINTER(c_float), POINTER(c_float), c_void_p]),
    "hb_orthonormalize_workspace_bytes": (ctypes.c_int, [c_int64, c_int64, POINTER(c_int64)]),
    "hb_orthonormalize_f32": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
    "hb_orthonormalize_f32_batched": (ctypes.c_int, [c_int32, POINTER(c_void_p), c_int64, c_int64, c_int64, POINTER(c_void_p), c_int64,
                                                     POINTER(c_void_p), c_void_p]),
    "hb_adam_precond": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_float, c_float, c_float, c_float, c_float, c_void_p]),
    "hb_adam_precond_grouped": (ctypes.c_int, [c_int32, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64),
                                               c_float, c_float, c_float, c_float, c_float, c_void_p]),
    "hb_copy_probe": (ctypes.c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "hb_last_error": (c_char_p, []),
    "hb_chunk_elems": (ctypes.c_int, []),
    "hb_abi_version": (ctypes.c_int, []),
}

_lib = None


class HbError(RuntimeError):
    pass


def prototypes():
    """name -> (restype, argtypes) of every exported entry point; tests check the library against it."""
    return dict(_PROTOTYPES)


def register(extra):
    """Other modules of the package add the entry points they bind (Muon, SOAP)."""
    _PROTOTYPES.update(extra)
    if _lib is not None:
        _bind(_lib, extra)


def _bind(lib, protos):
    for name, (res, args) in protos.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing: fail loudly
        fn.restype = res
        fn.argtypes = args


def lib():
    """The loaded library.  Raises HbError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HbError(
                f"{LIB_PATH} is missing: build it with `make -C heavyball_amd/csrc` (or __graft_entry__.build()). "
                "There is no CPU or PyTorch fallback for the optimizer step."
            )
        handle = ctypes.CDLL(LIB_PATH)
        _bind(handle, _PROTOTYPES)
        built = handle.hb_abi_version()
        if built != ABI_VERSION:
            raise HbError(f"{LIB_PATH} has ABI version {built}, this binding expects {ABI_VERSION}: rebuild it with `make -C heavyball_amd/csrc`")
        _lib = handle
    return _lib


def check(rc, what=""):
    if rc != 0:
        msg = lib().hb_last_error()
        raise HbError(f"{what or 'libhbstep'} failed with code {rc}: {msg.decode() if msg else ''}")


def chunk_elems():
    """HB_CHUNK of include/hbstep.h; tests assert that the built library agrees (hb_chunk_elems())."""
    return 4096

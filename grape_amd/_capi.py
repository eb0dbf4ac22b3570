"""ctypes binding of the C ABI declared in include/grape_hip.h.

The library must have been built (``python -m grape_amd.build``); loading fails loudly
otherwise — there is no fallback implementation of any kind.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# One curve per process, fixed when the library is compiled: GRAPE_CURVE = bls12_381 (default) or
# bn254 picks which build is loaded.
CURVE = os.environ.get("GRAPE_CURVE", "bls12_381")
if CURVE not in ("bls12_381", "bn254"):
    raise ValueError("GRAPE_CURVE must be bls12_381 or bn254, not %r" % CURVE)
LIB_PATH = os.path.join(_HERE, "libgrape_hip_bn254.so" if CURVE == "bn254" else "libgrape_hip.so")
FP_WORDS = 8 if CURVE == "bn254" else 12      # 32-bit words of an Fp element in memory

c_void_p = ctypes.c_void_p
c_size_t = ctypes.c_size_t
c_u32 = ctypes.c_uint32
c_i32 = ctypes.c_int32
c_int = ctypes.c_int

# name -> argument types (all functions return int unless listed in _RESTYPES)
SIGNATURES = {
    "grape_init": [c_int],
    "grape_last_error": [],
    "grape_stream_sync": [c_void_p],
    "grape_malloc": [ctypes.POINTER(c_void_p), c_size_t],
    "grape_free": [c_void_p],
    "grape_alloc_cache_release": [c_void_p],
    "grape_memcpy_h2d": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_memcpy_d2h": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_memcpy_d2d": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_memset_zero": [c_void_p, c_size_t, c_void_p],
    "grape_fr_add": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_sub": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_mul": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_bcast_add": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_bcast_mul": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_from_i32": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_from_u32": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_to_mont": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_from_mont": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_batch_inverse": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_shift_inverse": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_sum": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_sum_by_dim": [c_void_p, c_void_p, c_size_t, c_size_t, c_void_p],
    "grape_fr_pad": [c_void_p, c_void_p, c_u32, c_u32, c_size_t, c_void_p, c_void_p],
    "grape_i32_pad": [c_void_p, c_void_p, c_u32, c_u32, c_size_t, c_void_p],
    "grape_i32_pad_fill": [c_void_p, c_void_p, c_u32, c_u32, c_size_t, c_i32, c_void_p],
    "grape_fr_fold": [c_void_p, c_size_t, c_void_p, c_u32, c_u32, c_u32, c_void_p],
    "grape_fr_fold_i32_elems": [c_size_t, c_u32, c_u32],
    "grape_fr_fold_i32": [c_void_p, c_void_p, c_size_t, c_void_p, c_u32, c_u32, c_u32, c_void_p],
    "grape_sumcheck_round2": [c_void_p, c_void_p, c_u32, c_u32, c_void_p, c_void_p, c_void_p],
    "grape_sumcheck_round2_claim": [c_void_p, c_void_p, c_u32, c_u32, c_void_p, c_void_p, c_void_p, c_void_p],
    "grape_sumcheck_round2_noalloc": [c_void_p, c_void_p, c_u32, c_u32, c_void_p, c_void_p, c_void_p],
    "grape_sumcheck_round2_tail": [c_void_p, c_void_p, c_u32, c_u32, c_void_p, c_void_p, c_void_p],
    "grape_sumcheck_round2_coeffs": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u32, c_u32, c_void_p, c_void_p, c_void_p],
    "grape_sumcheck_round1": [c_void_p, c_void_p, c_void_p, c_u32, c_u32, c_void_p, c_void_p],
    "grape_eq_pyramid_elems": [c_u32],
    "grape_eq_pyramid": [c_void_p, c_void_p, c_u32, c_void_p],
    "grape_wround2": [c_void_p, c_void_p, c_void_p, c_void_p, c_u32, c_u32, c_u32, c_u32, c_void_p, c_int, c_void_p, c_void_p],
    "grape_wround2_partial_bytes": [c_u32],
    "grape_fold_tables": [c_void_p, c_void_p, c_u32, c_void_p],
    "grape_wround2_queue": [c_void_p, c_void_p, c_void_p, c_void_p, c_u32, c_u32, c_u32, c_u32, c_void_p, c_int, c_void_p, c_void_p, c_void_p],
    "grape_wround2_queue_indexed": [c_void_p, c_void_p, c_void_p, c_void_p, c_u32, c_void_p, c_void_p, c_u32, c_void_p, c_void_p, c_void_p, c_void_p],
    "grape_wround2_finish": [c_void_p, c_void_p, c_u32, c_int, c_void_p],
    "grape_sumcheck_round2_seg": [c_void_p, c_void_p, c_u32, c_u32, c_u32, c_void_p, c_void_p, c_void_p, c_void_p],
    "grape_wsum1_multi": [c_void_p, ctypes.POINTER(c_void_p), c_u32, c_u32, c_u32, c_void_p, c_void_p],
    "grape_tlookup_hist": [c_void_p, c_void_p, c_size_t, c_i32, c_u32, c_void_p],
    "grape_tlookup_index": [c_void_p, c_void_p, c_size_t, c_i32, c_u32, c_void_p],
    "grape_tlookup_hist_index": [c_void_p, c_void_p, c_size_t, c_u32, c_void_p],
    "grape_tlookup_inverse_by_table": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_u32, ctypes.POINTER(c_size_t), c_void_p],
    "grape_tlookup_index_inverse": [c_void_p, c_void_p, c_void_p, c_size_t, c_i32, c_u32, c_void_p, c_void_p, c_void_p, ctypes.POINTER(c_size_t), c_void_p],
    "grape_tlookup_index_embed_i32_nowait": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_i32, c_u32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "grape_tlookup_index_inverse_nowait": [c_void_p, c_void_p, c_void_p, c_size_t, c_i32, c_u32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "grape_fr_axpy": [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_tlookup_hot_select": [c_void_p, c_u32, c_u32, c_u32, c_void_p, c_void_p, ctypes.POINTER(ctypes.c_uint64), c_void_p],
    "grape_tlookup_hot_index": [c_void_p, c_void_p, c_size_t, c_void_p, c_u32, c_void_p],
    "grape_tlookup_hot_coverage": [c_void_p, c_u32, c_void_p, ctypes.POINTER(ctypes.c_uint64), c_void_p],
    "grape_fr_mask_cold": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_fr_gather": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_commit_fr_sparse": [c_void_p, c_void_p, c_void_p, c_size_t, c_u32, c_void_p, c_size_t, c_u32, c_u32, c_u32, c_void_p],
    "grape_g1_affine_add": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_tlookup_init": [c_void_p, c_void_p, c_i32, c_u32, c_void_p, c_void_p, c_void_p, c_void_p],
    "grape_tlookup_poly": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_tlookup_poly_sum": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_tlookup_round_sums": [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p],
    "grape_tlookup_mb_sums": [c_void_p, c_void_p, c_size_t, c_void_p, c_void_p],
    "grape_tlookup_table_round": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p],
    "grape_eq_table": [c_void_p, c_void_p, c_u32, c_void_p],
    "grape_eq_table_halve": [c_void_p, c_size_t, c_void_p],
    "grape_fr_fold_msb_multi": [ctypes.POINTER(c_void_p), c_u32, c_size_t, c_void_p, c_void_p],
    "grape_g1_generator": [c_void_p],
    "grape_g1_scalar_mul_base": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_g1_table_gen": [c_void_p, c_void_p, c_size_t, c_u32, c_void_p],
    "grape_g1_wide_table_gen": [c_void_p, c_void_p, c_size_t, c_u32, c_u32, c_u32, c_void_p],
    "grape_g1_wide_table_bytes": [c_size_t, c_u32, c_u32],
    "grape_g1_scaled_table_gen": [c_void_p, c_void_p, c_size_t, c_size_t, c_void_p, c_size_t, c_u32, c_u32, c_u32, c_void_p],
    "grape_commit_i32": [c_void_p, c_void_p, c_size_t, c_u32, c_void_p, c_size_t, c_u32, c_u32, c_u32, c_void_p],
    "grape_commit_i32_nowait": [c_void_p, c_void_p, c_size_t, c_u32, c_void_p, c_size_t, c_u32, c_u32, c_u32, c_void_p, c_void_p],
    "grape_commit_fr": [c_void_p, c_void_p, c_size_t, c_u32, c_void_p, c_size_t, c_u32, c_u32, c_u32, c_void_p],
    "grape_commit_fr_nowait": [c_void_p, c_void_p, c_size_t, c_u32, c_void_p, c_size_t, c_u32, c_u32, c_u32, c_void_p, c_void_p],
    "grape_g1_strided_table_gen": [c_void_p, c_void_p, c_size_t, c_u32, c_u32, c_u32, c_void_p],
    "grape_commit_fr_strided": [c_void_p, c_void_p, c_size_t, c_u32, c_void_p, c_size_t, c_u32, c_u32, c_u32, c_void_p],
    "grape_commit_i32_ref_table": [c_void_p, c_void_p, c_size_t, c_u32, c_void_p, c_size_t, c_void_p],
    "grape_commit_fr_ref_table": [c_void_p, c_void_p, c_size_t, c_u32, c_void_p, c_size_t, c_void_p],
    "grape_g1_affine_to_jacobian": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_g1_jacobian_to_affine": [c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_wit_matmul_rescale": [c_void_p, c_void_p, c_void_p, c_void_p, c_u32, c_u32, c_u32, c_u32, ctypes.c_int64, c_int, c_void_p],
    "grape_wit_set_matmul_method": [c_int],
    "grape_wit_elemul_rescale": [c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, ctypes.c_int64, c_void_p],
    "grape_wit_table_lookup": [c_void_p, c_void_p, c_size_t, c_i32, c_u32, c_void_p, c_void_p],
    "grape_wit_add_i32": [c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    "grape_wit_softmax": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u32, c_u32, c_void_p, c_u32, c_u32,
                          ctypes.c_int64, c_void_p],
    "grape_wit_row_sumsq": [c_void_p, c_void_p, c_u32, c_u32, c_void_p],
    "grape_wit_rmsnorm_apply": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u32, c_u32, ctypes.c_int64, c_void_p],
    "grape_wit_status": [ctypes.POINTER(c_u32), c_void_p],
    "grape_bench_copy": [c_void_p, c_void_p, c_size_t, c_int, ctypes.POINTER(ctypes.c_float), c_void_p],
    "grape_bench_copy_fr": [c_void_p, c_void_p, c_size_t, c_int, ctypes.POINTER(ctypes.c_float), c_void_p],
    "grape_bench_mad_u64_u32": [c_int, c_int, c_int, ctypes.POINTER(ctypes.c_double), c_void_p],
    "grape_profile_enable": [c_int],
    "grape_profile_last": [ctypes.POINTER(ctypes.c_float), c_int, ctypes.POINTER(c_int)],
    "grape_stream_create": [ctypes.POINTER(c_void_p)],
    "grape_stream_destroy": [c_void_p],
    "grape_stream_wait_event": [c_void_p, c_void_p],
    "grape_event_create": [ctypes.POINTER(c_void_p)],
    "grape_event_destroy": [c_void_p],
    "grape_event_record": [c_void_p, c_void_p],
    "grape_event_elapsed_ms": [ctypes.POINTER(ctypes.c_float), c_void_p, c_void_p],
}
_RESTYPES = {"grape_last_error": ctypes.c_char_p, "grape_g1_wide_table_bytes": c_size_t, "grape_eq_pyramid_elems": c_size_t,
             "grape_wround2_partial_bytes": c_size_t, "grape_fr_fold_i32_elems": c_size_t}

_lib = None


class GrapeError(RuntimeError):
    pass


def load():
    """Load the kernel library of the chosen curve and declare every entry point; raises if the library is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise GrapeError("%s not found: build it with `python -m grape_amd.build` "
                             "(there is no CPU fallback)" % LIB_PATH)
        # torch ships its own HIP runtime; when both live in one process the kernel library must
        # bind to the one torch has loaded, or the two runtimes fight over the device
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        lib = ctypes.CDLL(LIB_PATH)
        for name, args in SIGNATURES.items():
            fn = getattr(lib, name)     # AttributeError if a declared symbol is not exported
            fn.argtypes = args
            fn.restype = _RESTYPES.get(name, c_int)
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        raise GrapeError("grape_hip error %d: %s" % (rc, load().grape_last_error().decode()))

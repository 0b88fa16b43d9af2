"""ctypes binding of ``libbmtk_amd.so`` (declarations mirror ``include/bmtk_amd.h``).

There is no fallback: if the library cannot be loaded every compute entry
point raises.  ``load()`` compiles it once if the file is missing.
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libbmtk_amd.so")
_lib = None

c_void_p, c_int32, c_int64, c_float, c_double = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_double


class Glif3Sim(C.Structure):
    """``bmtk_glif3_sim`` of include/bmtk_amd.h, field for field."""
    _fields_ = [
        ("n_neurons", c_int64), ("batch", c_int32), ("ring_slots", c_int32), ("h", c_float), ("_pad0", c_int32),
        ("V", c_void_p), ("asc", c_void_p), ("y1", c_void_p), ("y2", c_void_p), ("ref", c_void_p),
        ("prop", c_void_p), ("prop_stride", c_int64), ("class_id", c_void_p), ("ring", c_void_p),
        ("rec_indptr", c_void_p), ("rec_indices", c_void_p), ("rec_weights", c_void_p),
        ("rec_delays", c_void_p), ("rec_receptors", c_void_p), ("rec_packed", c_void_p),
        ("n_inputs", c_int64), ("in_ptr", c_void_p), ("in_events", c_void_p),
        ("inp_indptr", c_void_p), ("inp_indices", c_void_p), ("inp_weights", c_void_p),
        ("inp_delays", c_void_p), ("inp_receptors", c_void_p), ("inp_packed", c_void_p), ("i_ext", c_void_p),
        ("work_bits", c_void_p), ("delay_offset", c_int32), ("hist_slots", c_int32),
        ("delay_bits", c_int32), ("res_spin_limit", C.c_uint32),
        ("res_span", c_int32), ("res_groups", c_int32), ("rec_seg", c_void_p), ("inp_seg", c_void_p),
        ("res_sync", c_void_p), ("res_fired", c_void_p),
        ("pull_indptr", c_void_p), ("pull_packed", c_void_p), ("pull_syn", c_void_p), ("pull_work", c_void_p),
        ("pull_inp_indptr", c_void_p), ("pull_inp_packed", c_void_p), ("pull_inp_syn", c_void_p),
        ("pull_inp_work", c_void_p), ("in_hist", c_void_p), ("in_hist_stride", c_int64),
        ("in_repeat_ptr", c_void_p), ("in_repeat_events", c_void_p),
        ("fuse_indptr", c_void_p), ("fuse_packed", c_void_p), ("fuse_any", c_void_p),
        ("fuse_hist_stride", c_int64), ("fuse_in_base", c_int64), ("fuse_shift", c_int32), ("fuse_wg_per_cu", c_int32),
        ("spike_bits", c_void_p), ("spike_bits_stride", c_int64),
        ("save_v", c_void_p), ("save_flags", c_void_p),
        ("probe_col", c_void_p), ("probe_v", c_void_p), ("probe_stride", c_int64), ("probe_every", c_int32),
        ("_pad1", c_int32),
        ("spike_step", c_void_p), ("spike_elem", c_void_p), ("spike_frac", c_void_p),
        ("spike_cap", c_int64), ("spike_count", c_void_p), ("spike_ways", c_int32), ("_pad2", c_int32),
    ]


class Glif3Bwd(C.Structure):
    """``bmtk_glif3_bwd`` of include/bmtk_amd.h, field for field."""
    _fields_ = [
        ("n_neurons", c_int64), ("batch", c_int32), ("ring_slots", c_int32), ("h", c_float), ("dampening", c_float),
        ("prop", c_void_p), ("prop_stride", c_int64), ("class_id", c_void_p),
        ("save_v", c_void_p), ("save_flags", c_void_p), ("spike_bits", c_void_p), ("spike_bits_stride", c_int64),
        ("rec_indptr", c_void_p), ("rec_packed", c_void_p),
        ("in_ptr", c_void_p), ("in_events", c_void_p), ("inp_indptr", c_void_p), ("inp_packed", c_void_p),
        ("dl_dz", c_void_p), ("dl_dz_const", c_void_p),
        ("lam_V", c_void_p), ("lam_asc", c_void_p), ("lam_y1", c_void_p), ("lam_y2", c_void_p),
        ("lam_ring", c_void_p), ("gz", c_void_p),
        ("d_rec_w", c_void_p), ("d_inp_w", c_void_p),
        ("blk_count", c_int32), ("gz_planes", c_int32), ("blk_indptr", c_void_p), ("blk_packed", c_void_p),
        ("d_blk_w", c_void_p),
    ]


ABI_VERSION = 24  # BMTK_AMD_ABI_VERSION of include/bmtk_amd.h that the mirrors above were written for

# name -> (restype, argtypes); every symbol include/bmtk_amd.h declares
SIGNATURES = {
    "bmtk_amd_abi_version": (c_int32, []),
    "bmtk_amd_last_error": (C.c_char_p, []),
    "bmtk_glif3_sim_sizeof": (c_int64, []),
    "bmtk_glif3_bwd_sizeof": (c_int64, []),
    "bmtk_glif3_precompute": (c_int32, [c_int64, c_void_p, c_double, c_void_p, c_void_p]),
    "bmtk_glif3_step_fwd": (c_int32, [c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_int64, c_void_p, c_float, c_void_p, c_int32, c_void_p,
                                      c_void_p, c_void_p, c_void_p, c_void_p]),
    "bmtk_spikes_compact_workspace_bytes": (c_int64, [c_int64]),
    "bmtk_spikes_compact": (c_int32, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "bmtk_spikes_compact_bits": (c_int32, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "bmtk_spikes_compact_noalloc": (c_int32, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "bmtk_csr_propagate_scatter": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p,
                                             c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_void_p]),
    "bmtk_csr_propagate_gather": (c_int32, [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_int32, c_int64, c_int64, c_void_p]),
    "bmtk_csr_propagate_auto_workspace_bytes": (c_int64, [c_int32, c_int64]),
    "bmtk_csr_propagate_auto": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int32, c_int64, c_int32] +
                                [c_void_p] * 7 + [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "bmtk_csr_propagate_auto2_workspace_bytes": (c_int64, [c_int32, c_int64]),
    "bmtk_csr_propagate_auto2": (c_int32, [c_void_p] * 4 + [c_int64, c_void_p, c_int64, c_int32, c_int64, c_int32] +
                                 [c_void_p] * 7 + [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "bmtk_csr_propagate_pull_workspace_bytes": (c_int64, [c_int32, c_int64]),
    "bmtk_csr_propagate_pull": (c_int32, [c_void_p, c_int64, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p,
                                          c_int64, c_int64, c_void_p, c_void_p]),
    "bmtk_csr_propagate_pull2": (c_int32, [c_void_p, c_int64, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p,
                                           c_int64, c_int64, c_void_p, c_void_p]),
    "bmtk_csr_pack": (c_int32, [c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "bmtk_csr_pack_wide": (c_int32, [c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p]),
    "bmtk_csr_segment_offsets": (c_int32, [c_int64, c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p,
                                           c_void_p]),
    "bmtk_poisson_count": (c_int32, [c_int64, c_int32, c_void_p, c_double, c_double, c_double, c_int64, C.c_uint64,
                                     c_void_p, c_void_p]),
    "bmtk_poisson_fill": (c_int32, [c_int64, c_int32, c_void_p, c_double, c_double, c_double, c_int64, C.c_uint64,
                                    c_void_p, c_void_p, c_void_p, c_void_p]),
    "bmtk_glif3_simulate_fwd": (c_int32, [C.POINTER(Glif3Sim), c_int64, c_int64, c_void_p]),
    "bmtk_glif3_simulate_bwd": (c_int32, [C.POINTER(Glif3Bwd), c_int64, c_int64, c_void_p]),
    "bmtk_glif3_step_bwd": (c_int32, [C.POINTER(Glif3Bwd), c_int64, c_int64, c_int32, c_void_p]),
    "bmtk_csr_weight_grad": (c_int32, [C.POINTER(Glif3Bwd), c_int64, c_int64, c_void_p]),
    "bmtk_csr_propagate_bwd": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_int32, c_int64, c_void_p,
                                         c_int32, c_void_p]),
    "bmtk_csr_propagate_bwd_blocked": (c_int32, [c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_int32, c_int64,
                                                 c_void_p, c_void_p]),
    "bmtk_csr_propagate_bwd_blocked_plan": (c_int32, [c_int64, c_int32, c_void_p]),
    "bmtk_microbench_lds": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "bmtk_microbench_atomics": (c_int32, [c_void_p, c_int64, c_int32, c_int32, c_int32, c_void_p]),
    "bmtk_microbench_hop": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, c_int32, C.c_uint32, c_void_p]),
    "bmtk_spike_counts": (c_int32, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
}


RES_SYNC_WORDS = (1 + 64 * 8) * 1088  # BMTK_RES_SYNC_WORDS
COMPACT_NOALLOC_MAX_N = 1 << 24       # BMTK_COMPACT_NOALLOC_MAX_N
RECORD_COUNT_STRIDE = 16
RES_FIRED_SLOTS = 16              # BMTK_RES_FIRED_SLOTS


class LibraryMissing(RuntimeError):
    pass


def load(build_if_missing=True):
    """Return the loaded library, compiling it first if the file is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        if not build_if_missing:
            raise LibraryMissing("{} not built; run `python -m bmtk_amd.csrc.build`".format(LIB_PATH))
        from .csrc.build import build
        build()
    try:
        lib = C.CDLL(LIB_PATH)
    except OSError as exc:
        raise LibraryMissing("cannot load {}: {}".format(LIB_PATH, exc))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    if lib.bmtk_amd_abi_version() != ABI_VERSION:
        raise LibraryMissing("{} has ABI version {}, these bindings are for {}; rebuild it".format(
            LIB_PATH, lib.bmtk_amd_abi_version(), ABI_VERSION))
    if lib.bmtk_glif3_sim_sizeof() != C.sizeof(Glif3Sim) or lib.bmtk_glif3_bwd_sizeof() != C.sizeof(Glif3Bwd):
        raise LibraryMissing("{} was built from a different include/bmtk_amd.h (struct size {} vs {}); rebuild it"
                             .format(LIB_PATH, lib.bmtk_glif3_sim_sizeof(), C.sizeof(Glif3Sim)))
    _lib = lib
    return lib


class BmtkAmdError(RuntimeError):
    pass


def check(code):
    if code != 0:
        msg = load().bmtk_amd_last_error()
        raise BmtkAmdError("libbmtk_amd error {}: {}".format(code, msg.decode() if msg else "?"))

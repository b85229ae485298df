"""ctypes view of libparamsp_hip.so (the C ABI declared in include/paramsp.h).

Used by the host-side format builder (row split, BCSR) and by tests / benchmarks that want to drive the
kernels without the PyTorch extension modules.  There is no fallback: if the library has not been built
the import of this module raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libparamsp_hip.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libparamsp_hip.so is not built: run `make -C %s` (or paramspmm_ae_amd/build_param.sh) first" % os.path.join(_HERE, "csrc")
    )

lib = ctypes.CDLL(LIB_PATH)

_vp = ctypes.c_void_p
_i = ctypes.c_int


class SpmmPlan(ctypes.Structure):
    _fields_ = [
        ("vec", _i),
        ("coarsen", _i),
        ("lanes_per_row", _i),
        ("rows_per_wave", _i),
        ("unroll", _i),
        ("col_tiles", _i),
        ("waves_per_block", _i),
        ("log_segs_per_wave", _i),
        ("even_split", _i),
        ("xcd_stripe_rows", _i),
    ]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_}


# name -> argtypes; the entries return int unless RESTYPES says otherwise.  Keep in step with include/paramsp.h.
SIGNATURES = {
    "psp_version": [],
    "psp_set_option": [ctypes.c_char_p, ctypes.c_longlong],
    "psp_get_option": [ctypes.c_char_p],
    "psp_spmm_plan_for": [_i, _i, _i, ctypes.POINTER(SpmmPlan)],
    "psp_spmm_register_sets": [_i, _i],
    "psp_split_csr_count": [_vp, _i, _i],
    "psp_split_csr": [_vp, _i, _i, _vp, _vp],
    "psp_split_csr_par": [_vp, _vp, _i, _i, _vp, _vp],
    "psp_bcsr_count": [_vp, _vp, _i, _i],
    "psp_bcsr_build": [_vp, _vp, _vp, _i, _i, _vp, _vp, _vp],
    "psp_scan_workspace_ints": [_i],
    "psp_split_csr_offsets_dev": [_vp, _i, _i, _vp, _vp, _i, _vp, _vp],
    "psp_split_csr_fill_dev": [_vp, _vp, _i, _i, _i, _vp, _vp, _vp],
    "psp_bcsr_offsets_dev": [_vp, _vp, _i, _vp, _vp, _i, _vp, _vp],
    "psp_bcsr_fill_dev": [_vp, _vp, _vp, _i, _vp, _vp, _vp, _vp],
    "psp_check_index_dev": [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp],
    "psp_vbsr_count": [_vp, _vp, _i, _i, _i],
    "psp_vbsr_build": [_vp, _vp, _vp, _i, _i, _i, _vp, _vp, _vp],
    "psp_spmm_act_f32": [_i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp],
    "psp_spmm_vec_f32": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "psp_spmm_vec_split_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "psp_genmask": [_vp, _vp, _vp, _i, _i, _vp, _vp],
    "psp_spmm_csr_f32": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "psp_spmm_csr_split_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "psp_spmm_bcsr_f32": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "psp_spmm_bcsr_split_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "psp_sddmm_csr_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "psp_sddmm_csr_split_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "psp_sddmm_csr_rowmax_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "psp_sddmm_csr_split_rowmax_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "psp_spmm_csr_softmax_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "psp_spmm_csr_split_softmax_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "psp_sddmm_bcsr_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "psp_sddmm_bcsr_split_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "psp_sddmm_vec_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "psp_sddmm_vec_split_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "psp_segment_softmax_f32": [_vp, _vp, _vp, _i, _vp],
    "psp_segment_softmax_ws_f32": [_vp, _vp, _vp, _i, _i, _vp, _vp],
    "psp_segment_softmax_static_f32": [_vp, _vp, _vp, _i, _i, _vp],
    "psp_spmm_f64": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "psp_sddmm_f64": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "psp_baseline_rowcache_spmm_f32": [_vp, _vp, _vp, _vp, _vp, _i, _i, _vp],
    "psp_nll_loss_stats_floats": [],
    "psp_nll_loss_mean_f32": [_vp, _vp, ctypes.c_longlong, _i, _vp, _vp, _vp],
    "psp_nll_loss_mean_backward_f32": [_vp, _vp, _vp, ctypes.c_longlong, _i, _vp, _vp],
    "psp_probe_gather_out_floats": [ctypes.c_longlong, _i, _i, _i],
    "psp_probe_gather_f32": [_vp, ctypes.c_longlong, _vp, _i, _i, _i, _i, _vp, ctypes.c_longlong, _vp],
    "psp_window_build": [_vp, _vp, _vp, _i, _vp, _vp, _vp],
    "psp_window_build_dev": [_vp, _vp, _vp, _i, _vp, _vp, _vp, _vp],
    "psp_spmm_window_plan": [_i, _i, ctypes.POINTER(_i), ctypes.POINTER(_i), ctypes.POINTER(_i)],
    "psp_spmm_window_f32": [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp],
    "psp_softmax_nll_supported": [_i],
    "psp_softmax_nll_mean_f32": [_vp, _vp, ctypes.c_longlong, _i, _vp, _vp, _vp],
    "psp_softmax_nll_mean_backward_f32": [_vp, _vp, _vp, _vp, ctypes.c_longlong, _i, _vp, _vp],
    "psp_sddmm_window_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "psp_attn_window_forward_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "psp_attn_window_backward_f32": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp],
    "psp_spmm_window_xw_f32": [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp],
    "psp_gemm_xw_supported": [_i, _i],
    "psp_gemm_xw_f32": [_vp, _vp, _vp, ctypes.c_longlong, _i, _i, _i, _vp],
    "psp_gemm_xw_act_f32": [_vp, _vp, _vp, ctypes.c_longlong, _i, _i, _i, _i, _vp, _vp],
    "psp_gemm_atb_ws_act_f32": [_vp, _vp, _vp, ctypes.c_longlong, _i, _i, _i, _vp, ctypes.c_longlong, _vp],
    "psp_gemm_atb_supported": [_i, _i],
    "psp_gemm_atb_f32": [_vp, _vp, _vp, ctypes.c_longlong, _i, _i, _vp],
    "psp_gemm_atb_workspace_floats": [ctypes.c_longlong, _i, _i],
    "psp_gemm_atb_ws_f32": [_vp, _vp, _vp, ctypes.c_longlong, _i, _i, _vp, ctypes.c_longlong, _vp],
}
# the entries that do not return int
RESTYPES = {"psp_gemm_atb_workspace_floats": ctypes.c_longlong, "psp_get_option": ctypes.c_longlong,
            "psp_probe_gather_out_floats": ctypes.c_longlong}

for _name, _args in SIGNATURES.items():
    _fn = getattr(lib, _name)
    _fn.argtypes = _args
    _fn.restype = RESTYPES.get(_name, _i)
lib.psp_last_error.argtypes = []
lib.psp_last_error.restype = ctypes.c_char_p

ABI_VERSION = 311  # PSP_ABI_VERSION of include/paramsp.h: the struct layouts and buffer sizes this module assumes
if lib.psp_version() < ABI_VERSION:
    raise ImportError("%s is version %d, this package needs %d: rebuild it (paramspmm_ae_amd/build_param.sh)"
                      % (LIB_PATH, lib.psp_version(), ABI_VERSION))


class ParamSpError(RuntimeError):
    pass


def check(rc):
    """Raise on a negative status; pass counts through."""
    if rc < 0:
        raise ParamSpError("libparamsp_hip: %s (status %d)" % (lib.psp_last_error().decode(), rc))
    return rc


CF_NATIVE = 1 << 16  # PSP_CF_NATIVE of include/paramsp.h


def pack_cf(coarsen, lanes, unroll=None, segs_per_wave=None, even_split=False):
    """Native SpMM configuration for the CF argument (PSP_CF_PACK): ``coarsen`` column vectors per lane, ``lanes``
    lanes per sparse row, ``unroll`` entries in flight (default: the largest with coarsen*unroll <= 4 ... 8 that the
    kernels are built for), ``segs_per_wave`` segments per wavefront (None = chosen by the library)."""
    if unroll is None:
        unroll = 4 if coarsen == 1 else 2 if coarsen <= 4 else 1
        unroll = min(unroll, lanes)
    log_l, log_u = lanes.bit_length() - 1, unroll.bit_length() - 1
    if 1 << log_l != lanes or 1 << log_u != unroll or not 1 <= coarsen <= 8 or lanes > 64 or unroll > 8:
        raise ValueError("pack_cf: coarsen 1..8, lanes and unroll powers of two (lanes <= 64, unroll <= 8)")
    sel = 0
    if segs_per_wave is not None:
        sel = segs_per_wave.bit_length()
        if 1 << (sel - 1) != segs_per_wave or sel > 7:
            raise ValueError("pack_cf: segs_per_wave must be a power of two up to 64")
    return CF_NATIVE | (coarsen - 1) | (log_l << 3) | (log_u << 6) | (sel << 8) | (int(bool(even_split)) << 11)


def unpack_cf(CF):
    """(coarsen, lanes, unroll, segs_per_wave or None, even_split) of a native CF value; None for a legacy CF."""
    if not CF & CF_NATIVE:
        return None
    sel = (CF >> 8) & 7
    return (CF & 7) + 1, 1 << ((CF >> 3) & 7), 1 << ((CF >> 6) & 3), (1 << (sel - 1)) if sel else None, bool(CF & (1 << 11))


def bw_stripe(rows):
    """Flag bits for the SpMM operators' blkWarpNum argument (PSP_BW_STRIPE): deal ``rows`` consecutive rows (segments)
    to one XCD at a time in this launch; 0 / None = the library option."""
    rows = int(rows or 0)
    if rows % 256 or not 0 <= rows <= 255 * 256:
        raise ValueError("bw_stripe: a multiple of 256 up to 65280")
    return (rows // 256) << 12


def set_option(name, value):
    check(lib.psp_set_option(name.encode(), int(value)))


def get_option(name):
    return check(lib.psp_get_option(name.encode()))


def spmm_plan(N, CF, blkWarpNum):
    p = SpmmPlan()
    check(lib.psp_spmm_plan_for(N, CF, blkWarpNum, ctypes.byref(p)))
    d = p.as_dict()
    d["register_sets"] = lib.psp_spmm_register_sets(p.unroll, p.lanes_per_row)  # which kernel variant the plan launches
    return d


def ptr(t):
    """Address of a torch tensor's / numpy array's first element (None -> NULL)."""
    if t is None:
        return None
    if hasattr(t, "data_ptr"):
        return t.data_ptr()
    return t.ctypes.data

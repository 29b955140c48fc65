"""ctypes binding of the C ABI declared in include/shflbw.h (libshflbw.so).

This is the FFI stub a maintainer of a Python caller would write; the tests and the
benchmark drive the library through it.  There is no fallback: if the shared library has
not been built, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libshflbw.so")
ARCHIVE_PATH = os.path.join(_HERE, "libblock_sparse.a")

# every symbol include/shflbw.h declares
EXPORTS = [
    "shflbw_status_string", "shflbw_last_error",
    "shflbw_random_mask_ex", "shflbw_random_mask",
    "shflbw_weight_create", "shflbw_weight_destroy",
    "shflbw_weight_init_random", "shflbw_filter_init_random", "shflbw_weight_set", "shflbw_weight_set_values",
    "shflbw_weight_dump_text", "shflbw_weight_load_text",
    "shflbw_weight_get_info", "shflbw_weight_host_arrays", "shflbw_weight_config_str",
    "shflbw_weight_sync_device", "shflbw_weight_meta_host", "shflbw_weight_device_ref",
    "shflbw_spmm_init", "shflbw_spmm_init_variant", "shflbw_spmm_exec",
    "shflbw_spmm_variant_count", "shflbw_spmm_variant_name",
    "shflbw_spconv_init", "shflbw_spconv_init_variant", "shflbw_spconv_exec",
    "shflbw_spconv_exec_static", "shflbw_spconv_init_chwb", "shflbw_spconv_host_reference_chwb",
    "shflbw_spconv_variant_count", "shflbw_spconv_variant_name", "shflbw_weight_release_scratch",
    "shflbw_spconv_check", "shflbw_weight_scratch_bytes",
    "shflbw_spmm_host_reference", "shflbw_spconv_host_reference",
    "shflbw_abi_sizes", "shflbw_device_info",
]

OK = 0
ERR_INVALID, ERR_SHAPE, ERR_STATE, ERR_HIP, ERR_UNSUPPORTED, ERR_FORMAT, ERR_CAPACITY = range(1, 8)
STATIC_SCRATCH_BYTES = 40 * 1024 * 1024  # SHFLBW_STATIC_SCRATCH_BYTES


class WeightInfo(C.Structure):
    _fields_ = [("nrow", C.c_int), ("ncol", C.c_int), ("nnzb", C.c_int), ("brow", C.c_int), ("bcol", C.c_int),
                ("density", C.c_float), ("seed", C.c_uint), ("row_permute", C.c_int),
                ("initialized", C.c_int), ("device_synced", C.c_int),
                ("F", C.c_int), ("R", C.c_int), ("S", C.c_int), ("C", C.c_int)]


class DeviceRef(C.Structure):
    _fields_ = [("meta", C.c_void_p), ("data", C.c_void_p), ("csb_indptr", C.c_void_p), ("csb_indices", C.c_void_p),
                ("row_permute_ids", C.c_void_p), ("csb_values", C.c_void_p)]


class _SpmmArgs(C.Structure):
    _fields_ = [("M", C.c_int), ("N", C.c_int), ("K", C.c_int), ("A_values", C.c_void_p), ("B", C.c_void_p),
                ("C", C.c_void_p), ("D", C.c_void_p), ("A_bsr_indptr", C.c_void_p), ("A_bsr_indices", C.c_void_p),
                ("A_row_indices", C.c_void_p), ("alpha", C.c_float), ("beta", C.c_float)]


class SpmmState(C.Structure):
    _fields_ = [("shared_mem_size", C.c_size_t), ("grid_dim", C.c_uint * 3), ("block_dim", C.c_uint * 3),
                ("init_success", C.c_int), ("variant", C.c_int), ("args", _SpmmArgs),
                ("packed_values", C.c_void_p), ("packed_indices", C.c_void_p), ("packed_indices_pm", C.c_void_p),
                ("panel_ptr", C.c_void_p), ("brow", C.c_int), ("ldb_bytes", C.c_int), ("zero_row", C.c_void_p),
                ("packed_slab", C.c_void_p)]


class _SpconvArgs(C.Structure):
    _fields_ = [("B", C.c_int), ("H", C.c_int), ("W", C.c_int), ("C", C.c_int), ("F", C.c_int), ("R", C.c_int),
                ("S", C.c_int), ("stride", C.c_int), ("A_values", C.c_void_p), ("IFMap", C.c_void_p),
                ("OFMap", C.c_void_p), ("A_bsr_indptr", C.c_void_p), ("A_bsr_indices", C.c_void_p),
                ("A_row_indices", C.c_void_p), ("alpha", C.c_float), ("beta", C.c_float)]


class SpconvState(C.Structure):
    _fields_ = [("shared_mem_size", C.c_size_t), ("grid_dim", C.c_uint * 3), ("block_dim", C.c_uint * 3),
                ("init_success", C.c_int), ("variant", C.c_int), ("args", _SpconvArgs),
                ("Ho", C.c_int), ("Wo", C.c_int),
                ("packed_values", C.c_void_p), ("packed_indices", C.c_void_p), ("panel_ptr", C.c_void_p),
                ("brow", C.c_int), ("result_fm", C.c_void_p), ("np", C.c_int),
                ("planes", C.c_void_p), ("plane_rows", C.c_int), ("plane_cols", C.c_int), ("plane_pitch", C.c_int),
                ("plane_copies", C.c_int), ("ncols", C.c_int), ("middle_tile_cols", C.c_int), ("xcds", C.c_int), ("cols_per_xcd", C.c_int), ("patience_ticks", C.c_int),
                ("sync", C.c_void_p), ("spmm", SpmmState)]


_lib = None


def load():
    """Load libshflbw.so; raises if the HIP extension has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libshflbw.so is missing (%s): build it with `make -C shflbw_sparse_nn_amd/csrc` "
            "or __graft_entry__.build(); there is no CPU fallback" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    vp, ci, cu, cf, sz = C.c_void_p, C.c_int, C.c_uint, C.c_float, C.c_size_t
    ip = C.POINTER(C.c_int)
    lib.shflbw_status_string.restype = C.c_char_p
    lib.shflbw_status_string.argtypes = [ci]
    lib.shflbw_last_error.restype = C.c_char_p
    lib.shflbw_random_mask_ex.argtypes = [ci, ci, ci, ci, cf, ci, ci, cu, ip, ip, vp, vp, sz]
    lib.shflbw_random_mask.argtypes = [ci, ci, ci, ci, cf, cu, ip, vp, vp, sz]
    lib.shflbw_weight_create.argtypes = [C.POINTER(vp)]
    lib.shflbw_weight_destroy.argtypes = [vp]
    lib.shflbw_weight_destroy.restype = None
    lib.shflbw_weight_init_random.argtypes = [vp, ci, ci, ci, ci, cf, ci, cu]
    lib.shflbw_filter_init_random.argtypes = [vp, ci, ci, ci, ci, ci, ci, cf, ci, cu]
    lib.shflbw_weight_set.argtypes = [vp, ci, ci, ci, ci, ci, vp, vp, vp, vp, ci, ci, ci]
    lib.shflbw_weight_set_values.argtypes = [vp, vp, sz]
    lib.shflbw_weight_dump_text.argtypes = [vp, C.c_char_p, sz, C.POINTER(sz)]
    lib.shflbw_weight_load_text.argtypes = [vp, C.c_char_p, sz]
    lib.shflbw_weight_get_info.argtypes = [vp, C.POINTER(WeightInfo)]
    lib.shflbw_weight_host_arrays.argtypes = [vp, C.POINTER(vp), C.POINTER(vp), C.POINTER(vp), C.POINTER(vp)]
    lib.shflbw_weight_config_str.restype = C.c_char_p
    lib.shflbw_weight_config_str.argtypes = [vp]
    lib.shflbw_weight_sync_device.argtypes = [vp]
    lib.shflbw_weight_meta_host.argtypes = [vp, C.POINTER(vp), C.POINTER(sz)]
    lib.shflbw_weight_device_ref.argtypes = [vp, C.POINTER(DeviceRef)]
    lib.shflbw_spmm_init.argtypes = [C.POINTER(SpmmState), vp, ci, vp, vp, vp, cf, cf]
    lib.shflbw_spmm_init_variant.argtypes = [C.POINTER(SpmmState), vp, ci, vp, vp, vp, cf, cf, ci]
    lib.shflbw_spmm_exec.argtypes = [C.POINTER(SpmmState), vp]
    lib.shflbw_spmm_variant_count.argtypes = [ci]
    lib.shflbw_spmm_variant_name.restype = C.c_char_p
    lib.shflbw_spmm_variant_name.argtypes = [ci, ci]
    lib.shflbw_spconv_init.argtypes = [C.POINTER(SpconvState), vp, ci, ci, ci, ci, vp, vp]
    lib.shflbw_spconv_init_variant.argtypes = [C.POINTER(SpconvState), vp, ci, ci, ci, ci, vp, vp, ci]
    lib.shflbw_spconv_exec.argtypes = [C.POINTER(SpconvState), vp]
    lib.shflbw_spconv_exec_static.argtypes = [vp, ci, ci, ci, ci, vp, vp, vp]
    lib.shflbw_spconv_init_chwb.argtypes = [C.POINTER(SpconvState), vp, ci, ci, ci, ci, vp, vp]
    lib.shflbw_spconv_host_reference_chwb.argtypes = [vp, ci, ci, ci, ci, vp, vp]
    lib.shflbw_spconv_variant_count.argtypes = []
    lib.shflbw_spconv_variant_name.restype = C.c_char_p
    lib.shflbw_spconv_variant_name.argtypes = [ci]
    lib.shflbw_weight_release_scratch.argtypes = [vp]
    lib.shflbw_spconv_check.argtypes = [C.POINTER(SpconvState)]
    lib.shflbw_weight_scratch_bytes.argtypes = [vp, C.POINTER(sz), ip]
    lib.shflbw_spmm_host_reference.argtypes = [vp, ci, vp, cf, vp, cf, vp]
    lib.shflbw_spconv_host_reference.argtypes = [vp, ci, ci, ci, ci, vp, vp]
    lib.shflbw_abi_sizes.restype = None
    lib.shflbw_abi_sizes.argtypes = [C.POINTER(sz), C.POINTER(sz)]
    lib.shflbw_device_info.argtypes = [ip, ip, C.POINTER(sz), C.c_char_p, sz]
    # the ctypes mirrors above must have the layout the library was compiled with
    a, b = sz(0), sz(0)
    lib.shflbw_abi_sizes(C.byref(a), C.byref(b))
    if (a.value, b.value) != (C.sizeof(SpmmState), C.sizeof(SpconvState)):
        raise RuntimeError("state struct layout mismatch: library %d/%d bytes, ctypes mirror %d/%d"
                           % (a.value, b.value, C.sizeof(SpmmState), C.sizeof(SpconvState)))
    _lib = lib
    return lib


class ShflbwError(RuntimeError):
    def __init__(self, status, detail):
        self.status = status
        super().__init__("shflbw status %d (%s): %s" % (status, load().shflbw_status_string(status).decode(), detail))


def check(status):
    if status != OK:
        raise ShflbwError(status, load().shflbw_last_error().decode())

"""Host-side mirror of the reference's operator interface, over the C ABI.

Same names, argument meaning and error behaviour as the reference's C++ classes so that the
parity tests read like the reference's own tests:
  BlockwiseSpMatrix   block_sparse/spmm/blockwise_format.h:13-68
  BlockwiseSpFilter   block_sparse/spconv/blockwise_format.h:17-27
  SpmmBlockwiseOp     block_sparse/spmm/blockwise_op.h:19-52
  SpconvBlockwiseOp   block_sparse/spconv/blockwise_op.h:19-48
Precondition violations the reference asserts on raise ShflbwError here.  Device buffers are
passed as integer device addresses (e.g. torch.Tensor.data_ptr()).
"""
import ctypes as C

import numpy as np

from . import capi


def _np_from(ptr, n, dtype):
    if n == 0 or not ptr:
        return np.zeros(0, dtype=dtype)
    buf = (C.c_char * (n * np.dtype(dtype).itemsize)).from_address(ptr)
    return np.frombuffer(buf, dtype=dtype).copy()


def random_mask(nrow, ncol, brow, bcol, block_density, seed, block_divisor=1, block_padding=1):
    """util/random_mask.h:4-10.  Returns (nnzb, indptr, indices[padded_nnzb])."""
    lib = capi.load()
    X = nrow // brow
    cap = int(nrow // brow * (ncol // bcol)) + X * block_padding + 8
    indptr = np.empty(X + 1, dtype=np.int32)
    indices = np.empty(cap, dtype=np.int32)
    nnzb, padded = C.c_int(0), C.c_int(0)
    capi.check(lib.shflbw_random_mask_ex(nrow, ncol, brow, bcol, block_density, block_divisor, block_padding, seed,
                                         C.byref(nnzb), C.byref(padded), indptr.ctypes.data, indices.ctypes.data, cap))
    return nnzb.value, indptr, indices[:padded.value].copy()


class BlockwiseSpMatrix:
    """Shfl-BW weight: row panels of `brow` rows, kept brow x 1 column vectors, optional row permutation."""

    def __init__(self):
        self._lib = capi.load()
        h = C.c_void_p()
        capi.check(self._lib.shflbw_weight_create(C.byref(h)))
        self._h = h

    def __del__(self):
        h = getattr(self, "_h", None)
        if h is not None and h.value:
            self._lib.shflbw_weight_destroy(h)
            self._h = None

    # -- construction -------------------------------------------------------------------
    def init_random(self, nrow, ncol, brow, bcol, expected_density, row_permute, seed):
        capi.check(self._lib.shflbw_weight_init_random(self._h, nrow, ncol, brow, bcol, expected_density,
                                                      int(bool(row_permute)), seed))

    def set(self, nrow, ncol, brow, bcol, indptr, indices, values, row_permute_ids=None, R=0, S=0, Cc=0):
        indptr = np.ascontiguousarray(indptr, dtype=np.int32)
        indices = np.ascontiguousarray(indices, dtype=np.int32)
        values = np.ascontiguousarray(values, dtype=np.float16).view(np.uint16)
        perm = None if row_permute_ids is None else np.ascontiguousarray(row_permute_ids, dtype=np.int32)
        if len(indptr) != nrow // max(brow, 1) + 1 or values.size != len(indices) * brow * bcol or (
                perm is not None and len(perm) != nrow):
            raise capi.ShflbwError(capi.ERR_SHAPE, "array lengths do not match the shape")
        capi.check(self._lib.shflbw_weight_set(self._h, nrow, ncol, brow, bcol, len(indices), indptr.ctypes.data,
                                               indices.ctypes.data, values.ctypes.data,
                                               None if perm is None else perm.ctypes.data, R, S, Cc))

    def set_values(self, values):
        values = np.ascontiguousarray(values, dtype=np.float16).view(np.uint16)
        capi.check(self._lib.shflbw_weight_set_values(self._h, values.ctypes.data, values.size))

    def load(self, text):
        b = text.encode() if isinstance(text, str) else text
        capi.check(self._lib.shflbw_weight_load_text(self._h, b, len(b)))

    def dump(self):
        need = C.c_size_t(0)
        capi.check(self._lib.shflbw_weight_dump_text(self._h, None, 0, C.byref(need)))
        buf = C.create_string_buffer(need.value)
        capi.check(self._lib.shflbw_weight_dump_text(self._h, buf, need.value, C.byref(need)))
        return buf.raw[:need.value].decode()

    def transform_and_sync_device(self):
        capi.check(self._lib.shflbw_weight_sync_device(self._h))

    # -- inspection ---------------------------------------------------------------------
    @property
    def info(self):
        i = capi.WeightInfo()
        capi.check(self._lib.shflbw_weight_get_info(self._h, C.byref(i)))
        return i

    def __getattr__(self, name):
        if name in ("nrow", "ncol", "nnzb", "brow", "bcol", "density", "seed", "F", "R", "S", "C"):
            return getattr(self.info, name)
        if name in ("row_permute", "initialized", "device_synced"):
            return bool(getattr(self.info, name))
        raise AttributeError(name)

    def _arrays(self):
        p = [C.c_void_p() for _ in range(4)]
        capi.check(self._lib.shflbw_weight_host_arrays(self._h, *[C.byref(x) for x in p]))
        i = self.info
        X = i.nrow // i.brow
        return (_np_from(p[0].value, X + 1, np.int32), _np_from(p[1].value, i.nnzb, np.int32),
                _np_from(p[2].value, i.nnzb * i.brow * i.bcol, np.uint16).view(np.float16),
                _np_from(p[3].value, i.nrow, np.int32) if p[3].value else None)

    @property
    def indptr(self):
        return self._arrays()[0]

    @property
    def indices(self):
        return self._arrays()[1]

    @property
    def values(self):
        return self._arrays()[2]

    @property
    def row_permute_ids(self):
        return self._arrays()[3]

    @property
    def config_str(self):
        return self._lib.shflbw_weight_config_str(self._h).decode()

    @property
    def meta_h(self):
        p, n = C.c_void_p(), C.c_size_t(0)
        capi.check(self._lib.shflbw_weight_meta_host(self._h, C.byref(p), C.byref(n)))
        return _np_from(p.value, n.value, np.int32)

    def host_reference(self, N, B, alpha=1.0, Cmat=None, beta=0.0):
        """get_host_reference (blockwise_format.h:268-311) computed by the library's host code: fp32 M x N."""
        B = np.ascontiguousarray(B, dtype=np.float16)
        Cm = None if Cmat is None else np.ascontiguousarray(Cmat, dtype=np.float16)
        out = np.empty((self.nrow, N), dtype=np.float32)
        capi.check(self._lib.shflbw_spmm_host_reference(self._h, N, B.ctypes.data, alpha,
                                                        None if Cm is None else Cm.ctypes.data, beta, out.ctypes.data))
        return out

    def release_scratch(self):
        capi.check(self._lib.shflbw_weight_release_scratch(self._h))

    @property
    def device_ref(self):
        r = capi.DeviceRef()
        capi.check(self._lib.shflbw_weight_device_ref(self._h, C.byref(r)))
        return r


class BlockwiseSpFilter(BlockwiseSpMatrix):
    """F x (R*S*C) filter matrix, column k = (r*S + s)*C + c."""

    def init_random(self, F, R, S, Cc, brow, bcol, expected_density, filter_permute, seed):
        capi.check(self._lib.shflbw_filter_init_random(self._h, F, R, S, Cc, brow, bcol, expected_density,
                                                      int(bool(filter_permute)), seed))

    def host_reference(self, x_nhwc, stride):
        """get_host_reference of the convolution (spconv/blockwise_format.h:55-132) over NHWC tensors: fp32
        [B][Ho][Wo][F]."""
        x = np.ascontiguousarray(x_nhwc, dtype=np.float16)
        Bn, H, W, _ = x.shape
        i = self.info
        Ho = (H + 2 * (i.R // 2) - i.R) // stride + 1
        Wo = (W + 2 * (i.S // 2) - i.S) // stride + 1
        out = np.empty((Bn, Ho, Wo, i.F), dtype=np.float32)
        capi.check(self._lib.shflbw_spconv_host_reference(self._h, Bn, H, W, stride, x.ctypes.data, out.ctypes.data))
        return out

    def host_reference_chwb(self, x_chwb, stride):
        """The same over the reference's tensors: input [C][H][W][B], output fp32 [F][H][W][B], H and W bounding both."""
        x = np.ascontiguousarray(x_chwb, dtype=np.float16)
        _, H, W, Bn = x.shape
        out = np.empty((self.info.F, H, W, Bn), dtype=np.float32)
        capi.check(self._lib.shflbw_spconv_host_reference_chwb(self._h, Bn, H, W, stride, x.ctypes.data, out.ctypes.data))
        return out


class SpmmBlockwiseOp:
    """initialize(spmat, N, B, [C,] D) then op() launches on `stream` (asynchronous)."""

    def __init__(self, variant=-1):
        self._lib = capi.load()
        self.variant = variant
        self._state = capi.SpmmState()

    def initialize(self, spmat, N, B, D, Cmat=None, alpha=1.0, beta=None):
        # the 4-argument form is alpha=1, beta=0; with C it is alpha=beta=1 (blockwise_op.h:143-159)
        if beta is None:
            beta = 0.0 if Cmat is None else 1.0
        capi.check(self._lib.shflbw_spmm_init_variant(C.byref(self._state), spmat._h, N, B, Cmat, D, alpha, beta,
                                                      self.variant))
        self._keep = spmat
        return self._state

    def __call__(self, stream=None):
        capi.check(self._lib.shflbw_spmm_exec(C.byref(self._state), stream))


class SpconvBlockwiseOp:
    """initialize(spfilter, B, H, W, stride, IFMap, OFMap); NHWC tensors, H and W are input extents.
    `variant` selects the form of the convolution (spconv_variants() names them); -1 is the library's choice."""

    def __init__(self, variant=-1):
        self._lib = capi.load()
        self._state = capi.SpconvState()
        self._variant = variant

    def initialize(self, spfilter, B, H, W, stride, IFMap, OFMap, batch_innermost=False):
        """batch_innermost=True: the reference's C-H-W-B / F-H-W-B tensors and its bounds rule (H, W bound input and
        output alike); the form is then fixed."""
        if batch_innermost:
            capi.check(self._lib.shflbw_spconv_init_chwb(C.byref(self._state), spfilter._h, B, H, W, stride, IFMap, OFMap))
        else:
            capi.check(self._lib.shflbw_spconv_init_variant(C.byref(self._state), spfilter._h, B, H, W, stride, IFMap,
                                                            OFMap, self._variant))
        self._keep = spfilter
        return self._state

    @property
    def output_hw(self):
        return self._state.Ho, self._state.Wo

    def __call__(self, stream=None):
        capi.check(self._lib.shflbw_spconv_exec(C.byref(self._state), stream))

    def check(self):
        """Waits for the device and raises if a launch of the fused form on this state did not run to completion."""
        capi.check(self._lib.shflbw_spconv_check(C.byref(self._state)))


def spmm_variants(brow):
    lib = capi.load()
    return [lib.shflbw_spmm_variant_name(brow, v).decode() for v in range(lib.shflbw_spmm_variant_count(brow))]


def spconv_variants():
    lib = capi.load()
    return [lib.shflbw_spconv_variant_name(v).decode() for v in range(lib.shflbw_spconv_variant_count())]


def spconv_variant_name(variant):
    return capi.load().shflbw_spconv_variant_name(variant).decode()


def device_info():
    lib = capi.load()
    cu, clk, lds = C.c_int(0), C.c_int(0), C.c_size_t(0)
    arch = C.create_string_buffer(64)
    capi.check(lib.shflbw_device_info(C.byref(cu), C.byref(clk), C.byref(lds), arch, 64))
    return dict(compute_units=cu.value, clock_khz=clk.value, lds_bytes=lds.value, arch=arch.value.decode())

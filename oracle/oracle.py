"""TEST INFRASTRUCTURE ONLY: ctypes loader for the CPU oracle (liboracle.so).

The oracle restates the reference's host algorithms (mask, permutation, value
generator, meta packing, SpMM and SpConv host references); see the citations in
shflbw_oracle.c.  Only tests, the smoke check and the benchmark's CPU-baseline
leg import this module; the shipped library never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = None

_I = C.c_int
_L = C.c_long
_F = C.c_float
_U = C.c_uint
_P = C.c_void_p


def build(force=False):
    """Compile liboracle.so (and _ref/ when the reference tree is present)."""
    so = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        _LIB = C.CDLL(so)
        _LIB.oracle_pack_meta.restype = _L
    return _LIB


def ref_lib():
    """The reference's own mask generator, if it was built in this container."""
    global _REF
    if _REF is None:
        so = os.path.join(_HERE, "_ref", "libref_mask.so")
        if not os.path.exists(so):
            return None
        _REF = C.CDLL(so)
    return _REF


def _ptr(a):
    return None if a is None else a.ctypes.data_as(_P)


def _i32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int32)


def _u16(a):
    """fp16 array -> its uint16 bit pattern (contiguous)."""
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return a.view(np.uint16)
    assert a.dtype == np.uint16, a.dtype
    return a


def shuffle_iota(n, seed):
    out = np.empty(n, dtype=np.int32)
    rc = lib().oracle_shuffle_iota(_I(n), _U(seed), _ptr(out))
    assert rc == 0
    return out


def row_permutation(nrow, seed):
    return shuffle_iota(nrow, seed)


def reference_values(n, skip=0):
    """(float)(rand() % 9 - 4) stream of an unseeded glibc rand()."""
    out = np.empty(n, dtype=np.float32)
    lib().oracle_reference_values(_L(skip), _L(n), _ptr(out))
    return out


def mask_nnzb(nrow, ncol, brow, bcol, density, divisor=1):
    return lib().oracle_mask_nnzb(_I(nrow), _I(ncol), _I(brow), _I(bcol), _F(density), _I(divisor))


def random_mask(nrow, ncol, brow, bcol, density, seed, divisor=1, padding=1):
    X = nrow // brow
    cap = mask_nnzb(nrow, ncol, brow, bcol, density, divisor) + X * padding + 8
    indptr = np.empty(X + 1, dtype=np.int32)
    indices = np.empty(cap, dtype=np.int32)
    nnzb = _I(0)
    padded = _I(0)
    rc = lib().oracle_random_mask_ex(_I(nrow), _I(ncol), _I(brow), _I(bcol), _F(density), _I(divisor), _I(padding),
                                     _U(seed), C.byref(nnzb), C.byref(padded), _ptr(indptr), _ptr(indices), _L(cap))
    assert rc == 0, rc
    return nnzb.value, indptr, indices[:padded.value].copy()


def ref_random_mask(nrow, ncol, brow, bcol, density, seed, divisor=1, padding=1):
    r = ref_lib()
    assert r is not None
    X = nrow // brow
    cap = mask_nnzb(nrow, ncol, brow, bcol, density, divisor) + X * padding + 8
    indptr = np.empty(X + 1, dtype=np.int32)
    indices = np.empty(cap, dtype=np.int32)
    nnzb = _I(0)
    padded = _I(0)
    rc = r.ref_random_mask(_I(nrow), _I(ncol), _I(brow), _I(bcol), _F(density), _I(divisor), _I(padding), _U(seed),
                           C.byref(nnzb), C.byref(padded), _ptr(indptr), _ptr(indices), _L(cap))
    assert rc == 0, rc
    return nnzb.value, indptr, indices[:padded.value].copy()


def pack_meta(nrow, brow, bcol, indptr, indices, perm):
    indptr, indices, perm = _i32(indptr), _i32(indices), _i32(perm)
    nnzb = len(indices)
    o1, o2 = _L(0), _L(0)
    total = lib().oracle_pack_meta(_I(nrow), _I(brow), _I(bcol), _I(nnzb), _ptr(indptr), _ptr(indices), _ptr(perm),
                                   None, C.byref(o1), C.byref(o2))
    meta = np.empty(total, dtype=np.int32)
    lib().oracle_pack_meta(_I(nrow), _I(brow), _I(bcol), _I(nnzb), _ptr(indptr), _ptr(indices), _ptr(perm),
                           _ptr(meta), C.byref(o1), C.byref(o2))
    return meta, o1.value, o2.value


def spmm_reference(nrow, ncol, brow, bcol, indptr, indices, values, perm, N, B, alpha=1.0, Cmat=None, beta=0.0,
                   nthreads=0):
    """fp32 D_ref (nrow x N) of the reference's get_host_reference for SpMM."""
    indptr, indices, perm = _i32(indptr), _i32(indices), _i32(perm)
    values, B, Cmat = _u16(values), _u16(B), _u16(Cmat)
    assert values.size == len(indices) * brow * bcol
    assert B.size == ncol * N
    D = np.empty((nrow, N), dtype=np.float32)
    rc = lib().oracle_spmm_reference(_I(nrow), _I(ncol), _I(brow), _I(bcol), _ptr(indptr), _ptr(indices), _ptr(values),
                                     _ptr(perm), _I(N), _ptr(B), _F(alpha), _ptr(Cmat), _F(beta), _ptr(D),
                                     _I(nthreads))
    assert rc == 0
    return D


def spconv_reference_chwb(F, R, S, Cc, brow, bcol, indptr, indices, values, perm, B, H, W, stride, ifmap):
    """fp32 output in the reference's F-H-W-B layout from C-H-W-B input."""
    indptr, indices, perm = _i32(indptr), _i32(indices), _i32(perm)
    values, ifmap = _u16(values), _u16(ifmap)
    out = np.empty((F, H, W, B), dtype=np.float32)
    rc = lib().oracle_spconv_reference_chwb(_I(F), _I(R), _I(S), _I(Cc), _I(brow), _I(bcol), _ptr(indptr),
                                            _ptr(indices), _ptr(values), _ptr(perm), _I(B), _I(H), _I(W), _I(stride),
                                            _ptr(ifmap), _ptr(out))
    assert rc == 0
    return out


def spconv_reference_nhwc(F, R, S, Cc, brow, indptr, indices, values, perm, B, H, W, stride, pad_h, pad_w, ifmap,
                          nthreads=0):
    """fp32 NHWC output (B, Ho, Wo, F) of a true strided, zero-padded sparse conv."""
    indptr, indices, perm = _i32(indptr), _i32(indices), _i32(perm)
    values, ifmap = _u16(values), _u16(ifmap)
    assert ifmap.size == B * H * W * Cc
    Ho = (H + 2 * pad_h - R) // stride + 1
    Wo = (W + 2 * pad_w - S) // stride + 1
    out = np.empty((B, Ho, Wo, F), dtype=np.float32)
    rc = lib().oracle_spconv_reference_nhwc(_I(F), _I(R), _I(S), _I(Cc), _I(brow), _ptr(indptr), _ptr(indices),
                                            _ptr(values), _ptr(perm), _I(B), _I(H), _I(W), _I(stride), _I(pad_h),
                                            _I(pad_w), _ptr(ifmap), _ptr(out), _I(nthreads))
    assert rc == 0
    return out


def half_to_float(h):
    h = _u16(h)
    out = np.empty(h.shape, dtype=np.float32)
    lib().oracle_half_to_float(_ptr(h), _ptr(out), _L(h.size))
    return out


def float_to_half(f):
    f = np.ascontiguousarray(f, dtype=np.float32)
    out = np.empty(f.shape, dtype=np.uint16)
    lib().oracle_float_to_half(_ptr(f), _ptr(out), _L(f.size))
    return out.view(np.float16)


def max_threads():
    return lib().oracle_max_threads()


# --------------------------------------------------------------------------
# text dump / load of a weight matrix: spmm/blockwise_format.h:125-198 and
# example/spmatrix_dump_load.md (whitespace separated numbers; '#' comments
# are only in the documentation's worked examples and are stripped here).
# --------------------------------------------------------------------------

def parse_dump(text):
    toks = []
    for line in text.splitlines():
        line = line.split("#", 1)[0]
        toks.extend(line.split())
    it = iter(toks)
    nrow, ncol, nnzb, brow, bcol, rp = (int(next(it)) for _ in range(6))
    X = nrow // brow
    indptr = np.array([int(next(it)) for _ in range(X + 1)], dtype=np.int32)
    indices = np.array([int(next(it)) for _ in range(nnzb)], dtype=np.int32)
    values = np.array([float(next(it)) for _ in range(nnzb * brow * bcol)], dtype=np.float32)
    perm = np.array([int(next(it)) for _ in range(nrow)], dtype=np.int32) if rp else None
    return dict(nrow=nrow, ncol=ncol, nnzb=nnzb, brow=brow, bcol=bcol, row_permute=bool(rp), indptr=indptr,
                indices=indices, values=values.astype(np.float16), row_permute_ids=perm)


def densify(m):
    """Dense logical matrix of a parsed/constructed weight (row i of the stored
    panels lands at logical row row_permute_ids[i]; values column-major per block)."""
    nrow, ncol, brow, bcol = m["nrow"], m["ncol"], m["brow"], m["bcol"]
    A = np.zeros((nrow, ncol), dtype=np.float32)
    vals = np.asarray(m["values"], dtype=np.float32).reshape(-1, bcol, brow)
    perm = m.get("row_permute_ids")
    for i in range(nrow // brow):
        for p in range(m["indptr"][i], m["indptr"][i + 1]):
            j = m["indices"][p] * bcol
            for kk in range(bcol):
                for mm in range(brow):
                    r = i * brow + mm
                    if perm is not None:
                        r = perm[r]
                    A[r, j + kk] = vals[p, kk, mm]
    return A

// Names of the entries of the operator tables (block_sparse/common/library_util.h:3-9): one
// pair of global function-pointer variables per tile configuration of the reference,
//   <Type>_<BM>x<BN>x<BK>_<WM>x<WN>x<WK>_<MM>x<MN>x<MK>_<NSTAGE>_{Init,Exec}Fn
#pragma once

#define NAME_FUN(type, fn, BM, BN, BK, WM, WN, WK, MM, MN, MK, NSTAGE) \
    type##_##BM##x##BN##x##BK##_##WM##x##WN##x##WK##_##MM##x##MN##x##MK##_##NSTAGE##_##fn##Fn

#define DECL_FUN(type, BM, BN, BK, WM, WN, WK, MM, MN, MK, NSTAGE)                       \
    extern type##InitFn_t NAME_FUN(type, Init, BM, BN, BK, WM, WN, WK, MM, MN, MK, NSTAGE); \
    extern type##ExecFn_t NAME_FUN(type, Exec, BM, BN, BK, WM, WN, WK, MM, MN, MK, NSTAGE);

// definition of one pair, both pointing at the per-block-height native entry
#define DEFN_FUN(type, BM, BN, BK, WM, WN, WK, MM, MN, MK, NSTAGE)                                         \
    type##InitFn_t NAME_FUN(type, Init, BM, BN, BK, WM, WN, WK, MM, MN, MK, NSTAGE) =                      \
        type##InitFn<ShapeBase<BM, BN, BK>, ShapeBase<WM, WN, WK>, ShapeBase<MM, MN, MK>, NSTAGE>;         \
    type##ExecFn_t NAME_FUN(type, Exec, BM, BN, BK, WM, WN, WK, MM, MN, MK, NSTAGE) =                      \
        type##ExecFn<ShapeBase<BM, BN, BK>, ShapeBase<WM, WN, WK>, ShapeBase<MM, MN, MK>, NSTAGE>;

// Declarations of the SpMM operator table (block_sparse/spmm/spmm_library_decl.h); the
// definitions live in blockwise_library.cc, archived into libblock_sparse.a.
#pragma once
#include "block_sparse/common/library_util.h"
#include "block_sparse/spmm/blockwise_op.h"

#define SHFLBW_TILE(...) DECL_FUN(SpmmBlockwise, __VA_ARGS__)
#include "block_sparse/common/library_table.def"
#undef SHFLBW_TILE

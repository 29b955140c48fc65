// Declarations of the SpConv operator table (block_sparse/spconv/spconv_library_decl.h); the
// definitions live in blockwise_library.cc, archived into libblock_sparse.a.
#pragma once
#include "block_sparse/common/library_util.h"
#include "block_sparse/spconv/blockwise_op.h"

#define SHFLBW_TILE(...) DECL_FUN(SpconvBlockwise, __VA_ARGS__)
#include "block_sparse/common/library_table.def"
#undef SHFLBW_TILE

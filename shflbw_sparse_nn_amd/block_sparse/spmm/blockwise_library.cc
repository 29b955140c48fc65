// Definitions of the SpMM operator table (block_sparse/spmm/blockwise_library.cu:13-223).
#include "block_sparse/spmm/spmm_library_decl.h"

#define SHFLBW_TILE(...) DEFN_FUN(SpmmBlockwise, __VA_ARGS__)
#include "block_sparse/common/library_table.def"
#undef SHFLBW_TILE

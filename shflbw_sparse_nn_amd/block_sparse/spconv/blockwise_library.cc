// Definitions of the SpConv operator table (block_sparse/spconv/blockwise_library.cu).
#include "block_sparse/spconv/spconv_library_decl.h"

#define SHFLBW_TILE(...) DEFN_FUN(SpconvBlockwise, __VA_ARGS__)
#include "block_sparse/common/library_table.def"
#undef SHFLBW_TILE

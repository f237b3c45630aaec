// map_cast_d.hip — cast rows for a group of source dtypes (nx_c_map.c:1003-1044).
#include "map_cast.hpp"

map_launch_fn nxh_lookup_cast_d(int src, int dst) {
  static const CastRow<NXH_I64> row_NXH_I64;
  static const CastRow<NXH_U64> row_NXH_U64;
  static const CastRow<NXH_C32> row_NXH_C32;
  static const CastRow<NXH_C64> row_NXH_C64;
  switch (src) {
    case NXH_I64: return row_NXH_I64.fn[dst];
    case NXH_U64: return row_NXH_U64.fn[dst];
    case NXH_C32: return row_NXH_C32.fn[dst];
    case NXH_C64: return row_NXH_C64.fn[dst];
    default: return nullptr;
  }
}

// map_cast_c.hip — cast rows for a group of source dtypes (nx_c_map.c:1003-1044).
#include "map_cast.hpp"

map_launch_fn nxh_lookup_cast_c(int src, int dst) {
  static const CastRow<NXH_I16> row_NXH_I16;
  static const CastRow<NXH_U16> row_NXH_U16;
  static const CastRow<NXH_I32> row_NXH_I32;
  static const CastRow<NXH_U32> row_NXH_U32;
  switch (src) {
    case NXH_I16: return row_NXH_I16.fn[dst];
    case NXH_U16: return row_NXH_U16.fn[dst];
    case NXH_I32: return row_NXH_I32.fn[dst];
    case NXH_U32: return row_NXH_U32.fn[dst];
    default: return nullptr;
  }
}

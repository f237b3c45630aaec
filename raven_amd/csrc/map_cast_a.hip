// map_cast_a.hip — cast rows for a group of source dtypes (nx_c_map.c:1003-1044).
#include "map_cast.hpp"

map_launch_fn nxh_lookup_cast_a(int src, int dst) {
  static const CastRow<NXH_F16> row_NXH_F16;
  static const CastRow<NXH_F32> row_NXH_F32;
  static const CastRow<NXH_F64> row_NXH_F64;
  static const CastRow<NXH_BF16> row_NXH_BF16;
  switch (src) {
    case NXH_F16: return row_NXH_F16.fn[dst];
    case NXH_F32: return row_NXH_F32.fn[dst];
    case NXH_F64: return row_NXH_F64.fn[dst];
    case NXH_BF16: return row_NXH_BF16.fn[dst];
    default: return nullptr;
  }
}

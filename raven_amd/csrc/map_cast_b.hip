// map_cast_b.hip — cast rows for a group of source dtypes (nx_c_map.c:1003-1044).
#include "map_cast.hpp"

map_launch_fn nxh_lookup_cast_b(int src, int dst) {
  static const CastRow<NXH_F8E4M3> row_NXH_F8E4M3;
  static const CastRow<NXH_F8E5M2> row_NXH_F8E5M2;
  static const CastRow<NXH_I8> row_NXH_I8;
  static const CastRow<NXH_U8> row_NXH_U8;
  static const CastRow<NXH_BOOL> row_NXH_BOOL;
  switch (src) {
    case NXH_F8E4M3: return row_NXH_F8E4M3.fn[dst];
    case NXH_F8E5M2: return row_NXH_F8E5M2.fn[dst];
    case NXH_I8: return row_NXH_I8.fn[dst];
    case NXH_U8: return row_NXH_U8.fn[dst];
    case NXH_BOOL: return row_NXH_BOOL.fn[dst];
    default: return nullptr;
  }
}

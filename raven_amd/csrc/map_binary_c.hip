// map_binary_c.hip — binary elementwise ops, one dispatch row per op (nx_c_map.c:494-695, stubs :1207-1219).
#include "map_ops.hpp"

map_launch_fn nxh_lookup_binary_c(int op, int dt) {
  static const MapRowOf<BinaryF, OpPow> row_OpPow;
  static const MapRowOf<BinaryF, OpAtan2> row_OpAtan2;
  static const MapRowOf<BinaryF, OpXor> row_OpXor;
  static const MapRowOf<BinaryF, OpOr> row_OpOr;
  static const MapRowOf<BinaryF, OpAnd> row_OpAnd;
  switch (op) {
    case NXH_POW: return row_OpPow.fn[dt];
    case NXH_ATAN2: return row_OpAtan2.fn[dt];
    case NXH_XOR: return row_OpXor.fn[dt];
    case NXH_OR: return row_OpOr.fn[dt];
    case NXH_AND: return row_OpAnd.fn[dt];
    default: return nullptr;
  }
}

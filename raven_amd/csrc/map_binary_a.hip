// map_binary_a.hip — binary elementwise ops, one dispatch row per op (nx_c_map.c:494-695, stubs :1207-1219).
#include "map_ops.hpp"

map_launch_fn nxh_lookup_binary_a(int op, int dt) {
  static const MapRowOf<BinaryF, OpAdd> row_OpAdd;
  static const MapRowOf<BinaryF, OpSub> row_OpSub;
  static const MapRowOf<BinaryF, OpMul> row_OpMul;
  static const MapRowOf<BinaryF, OpMax> row_OpMax;
  static const MapRowOf<BinaryF, OpMin> row_OpMin;
  switch (op) {
    case NXH_ADD: return row_OpAdd.fn[dt];
    case NXH_SUB: return row_OpSub.fn[dt];
    case NXH_MUL: return row_OpMul.fn[dt];
    case NXH_MAX: return row_OpMax.fn[dt];
    case NXH_MIN: return row_OpMin.fn[dt];
    default: return nullptr;
  }
}

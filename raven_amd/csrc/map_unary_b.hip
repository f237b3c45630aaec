// map_unary_b.hip — unary elementwise ops, one dispatch row per op (nx_c_map.c:300-488, stubs :1184-1204).
#include "map_ops.hpp"

map_launch_fn nxh_lookup_unary_b(int op, int dt) {
  static const MapRowOf<UnaryF, OpExp> row_OpExp;
  static const MapRowOf<UnaryF, OpLog> row_OpLog;
  static const MapRowOf<UnaryF, OpSin> row_OpSin;
  static const MapRowOf<UnaryF, OpCos> row_OpCos;
  switch (op) {
    case NXH_EXP: return row_OpExp.fn[dt];
    case NXH_LOG: return row_OpLog.fn[dt];
    case NXH_SIN: return row_OpSin.fn[dt];
    case NXH_COS: return row_OpCos.fn[dt];
    default: return nullptr;
  }
}

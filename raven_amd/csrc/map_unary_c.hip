// map_unary_c.hip — unary elementwise ops, one dispatch row per op (nx_c_map.c:300-488, stubs :1184-1204).
#include "map_ops.hpp"

map_launch_fn nxh_lookup_unary_c(int op, int dt) {
  static const MapRowOf<UnaryF, OpTan> row_OpTan;
  static const MapRowOf<UnaryF, OpAsin> row_OpAsin;
  static const MapRowOf<UnaryF, OpAcos> row_OpAcos;
  static const MapRowOf<UnaryF, OpAtan> row_OpAtan;
  switch (op) {
    case NXH_TAN: return row_OpTan.fn[dt];
    case NXH_ASIN: return row_OpAsin.fn[dt];
    case NXH_ACOS: return row_OpAcos.fn[dt];
    case NXH_ATAN: return row_OpAtan.fn[dt];
    default: return nullptr;
  }
}

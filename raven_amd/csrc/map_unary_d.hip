// map_unary_d.hip — unary elementwise ops, one dispatch row per op (nx_c_map.c:300-488, stubs :1184-1204).
#include "map_ops.hpp"

map_launch_fn nxh_lookup_unary_d(int op, int dt) {
  static const MapRowOf<UnaryF, OpSinh> row_OpSinh;
  static const MapRowOf<UnaryF, OpCosh> row_OpCosh;
  static const MapRowOf<UnaryF, OpTanh> row_OpTanh;
  static const MapRowOf<UnaryF, OpErf> row_OpErf;
  switch (op) {
    case NXH_SINH: return row_OpSinh.fn[dt];
    case NXH_COSH: return row_OpCosh.fn[dt];
    case NXH_TANH: return row_OpTanh.fn[dt];
    case NXH_ERF: return row_OpErf.fn[dt];
    default: return nullptr;
  }
}

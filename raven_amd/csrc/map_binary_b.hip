// map_binary_b.hip — binary elementwise ops, one dispatch row per op (nx_c_map.c:494-695, stubs :1207-1219).
#include "map_ops.hpp"

map_launch_fn nxh_lookup_binary_b(int op, int dt) {
  static const MapRowOf<BinaryF, OpIdiv> row_OpIdiv;
  static const MapRowOf<BinaryF, OpFdiv> row_OpFdiv;
  static const MapRowOf<BinaryF, OpMod> row_OpMod;
  switch (op) {
    case NXH_IDIV: return row_OpIdiv.fn[dt];
    case NXH_FDIV: return row_OpFdiv.fn[dt];
    case NXH_MOD: return row_OpMod.fn[dt];
    default: return nullptr;
  }
}

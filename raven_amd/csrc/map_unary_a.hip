// map_unary_a.hip — unary elementwise ops, one dispatch row per op (nx_c_map.c:300-488, stubs :1184-1204).
#include "map_ops.hpp"

map_launch_fn nxh_lookup_unary_a(int op, int dt) {
  static const MapRowOf<UnaryF, OpNeg> row_OpNeg;
  static const MapRowOf<UnaryF, OpRecip> row_OpRecip;
  static const MapRowOf<UnaryF, OpAbs> row_OpAbs;
  static const MapRowOf<UnaryF, OpSign> row_OpSign;
  static const MapRowOf<UnaryF, OpSqrt> row_OpSqrt;
  static const MapRowOf<UnaryF, OpTrunc> row_OpTrunc;
  static const MapRowOf<UnaryF, OpCeil> row_OpCeil;
  static const MapRowOf<UnaryF, OpFloor> row_OpFloor;
  static const MapRowOf<UnaryF, OpRound> row_OpRound;
  switch (op) {
    case NXH_NEG: return row_OpNeg.fn[dt];
    case NXH_RECIP: return row_OpRecip.fn[dt];
    case NXH_ABS: return row_OpAbs.fn[dt];
    case NXH_SIGN: return row_OpSign.fn[dt];
    case NXH_SQRT: return row_OpSqrt.fn[dt];
    case NXH_TRUNC: return row_OpTrunc.fn[dt];
    case NXH_CEIL: return row_OpCeil.fn[dt];
    case NXH_FLOOR: return row_OpFloor.fn[dt];
    case NXH_ROUND: return row_OpRound.fn[dt];
    default: return nullptr;
  }
}

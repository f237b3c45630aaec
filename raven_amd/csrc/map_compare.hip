// map_compare.hip — comparisons (bool output, dispatched on the input dtype;
// nx_c_map.c:746-803, 1231-1256), where (storage-typed select, :809-839) and the
// identity copy behind copy / contiguous / assign / full (nx_c_move.c:61-84).
#include "map_ops.hpp"

map_launch_fn nxh_lookup_compare(int op, int dt) {
  static const MapRowOf<CompareF, OpEq> row_eq;
  static const MapRowOf<CompareF, OpNe> row_ne;
  static const MapRowOf<CompareF, OpLt> row_lt;
  static const MapRowOf<CompareF, OpLe> row_le;
  switch (op) {
    case NXH_CMPEQ: return row_eq.fn[dt];
    case NXH_CMPNE: return row_ne.fn[dt];
    case NXH_CMPLT: return row_lt.fn[dt];
    case NXH_CMPLE: return row_le.fn[dt];
    default: return nullptr;
  }
}

// where and copy move storage bits untouched, so they are keyed by element
// size, not dtype.
struct alignas(16) B16 {
  uint64_t lo, hi;
};
template <class S>
struct WhereF {
  static constexpr int NIN = 3;
  using Out = S;
  using In0 = uint8_t;
  using In1 = S;
  using In2 = S;
  __device__ __forceinline__ static Out apply(In0 c, In1 a, In2 b) { return c ? a : b; }
};
template <class S>
struct CopyF {
  static constexpr int NIN = 1;
  using Out = S;
  using In0 = S;
  using In1 = Unused;
  using In2 = Unused;
  __device__ __forceinline__ static Out apply(In0 a) { return a; }
};

map_launch_fn nxh_lookup_where(int elem_size) {
  switch (elem_size) {
    case 1: return &map_launch<WhereF<uint8_t>>;
    case 2: return &map_launch<WhereF<uint16_t>>;
    case 4: return &map_launch<WhereF<uint32_t>>;
    case 8: return &map_launch<WhereF<uint64_t>>;
    case 16: return &map_launch<WhereF<B16>>;
    default: return nullptr;
  }
}
map_launch_fn nxh_lookup_copy(int elem_size) {
  switch (elem_size) {
    case 1: return &map_launch<CopyF<uint8_t>>;
    case 2: return &map_launch<CopyF<uint16_t>>;
    case 4: return &map_launch<CopyF<uint32_t>>;
    case 8: return &map_launch<CopyF<uint64_t>>;
    case 16: return &map_launch<CopyF<B16>>;
    default: return nullptr;
  }
}

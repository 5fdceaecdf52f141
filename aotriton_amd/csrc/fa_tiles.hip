// Compile-time tile/occupancy table keyed on (element type, head dim, causal / windowed), reported
// through fa_query_*_config.
#include "fa_fwd_impl.h"
#include "fa_bwd_impl.h"
#include "fa_kernels.h"

namespace fa {

template <typename T, int D, bool W> static TileShape fwd_shape() {
  using Tile = FwdTile<T, D, W>;
  return TileShape{Tile::BM, Tile::BN, Tile::NW, Tile::LDS};
}

template <typename T> static TileShape fwd_shape_of(int head_dim, bool windowed) {
  switch (head_dim) {
    case 64: return windowed ? fwd_shape<T, 64, true>() : fwd_shape<T, 64, false>();
    case 128: return windowed ? fwd_shape<T, 128, true>() : fwd_shape<T, 128, false>();
    default: return windowed ? fwd_shape<T, 256, true>() : fwd_shape<T, 256, false>();
  }
}

TileShape fwd_tile_shape(int dtype, int head_dim, bool windowed) {
  return dtype == kDtypeBF16 ? fwd_shape_of<bf16_t>(head_dim, windowed) : fwd_shape_of<f16_t>(head_dim, windowed);
}

template <typename T> static TileShape bwd_shape_of(int head_dim, bool windowed, int slot) {
  switch (head_dim) {
    case 64: return windowed ? bwd_shape<T, 64, true>(slot) : bwd_shape<T, 64, false>(slot);
    case 128: return windowed ? bwd_shape<T, 128, true>(slot) : bwd_shape<T, 128, false>(slot);
    default: return windowed ? bwd_shape<T, 256, true>(slot) : bwd_shape<T, 256, false>(slot);
  }
}

TileShape bwd_tile_shape(int dtype, int head_dim, bool windowed, int kernel_slot) {
  return dtype == kDtypeBF16 ? bwd_shape_of<bf16_t>(head_dim, windowed, kernel_slot)
                             : bwd_shape_of<f16_t>(head_dim, windowed, kernel_slot);
}

}  // namespace fa

// Compile-time tile/occupancy table, reported through fa_query_*_config.
#include "fa_fwd_impl.h"
#include "fa_bwd_impl.h"
#include "fa_kernels.h"

namespace fa {

template <int D> static TileShape fwd_shape() {
  return TileShape{FwdTile<D>::NW * 32, FwdTile<D>::BN, FwdTile<D>::NW, FwdSmem<D, FwdTile<D>::BN, FwdTile<D>::NW>::BYTES};
}

TileShape fwd_tile_shape(int head_dim) {
  switch (head_dim) {
    case 64: return fwd_shape<64>();
    case 128: return fwd_shape<128>();
    default: return fwd_shape<256>();
  }
}

TileShape bwd_tile_shape(int head_dim, int kernel_slot) {
  switch (head_dim) {
    case 64: return bwd_shape<64>(kernel_slot);
    case 128: return bwd_shape<128>(kernel_slot);
    default: return bwd_shape<256>(kernel_slot);
  }
}

}  // namespace fa

#pragma once
#include "fa_device.h"
#include "fa_kernels.h"
namespace fa {
template <int D> TileShape bwd_shape(int slot) { (void)slot; return TileShape{128, 128, 4, 0}; }
}

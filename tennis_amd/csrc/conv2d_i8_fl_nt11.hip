// Flat-tile int8 convolution kernel, tiles of 1 + 1 position fragments.
#define TSX_FL_NTA 1
#define TSX_FL_NTB 1
#include "conv2d_i8_fl_kernel.hpp"

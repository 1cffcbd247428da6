// Flat-tile int8 convolution kernel, tiles of 4 + 3 position fragments.
#define TSX_FL_NTA 4
#define TSX_FL_NTB 3
#include "conv2d_i8_fl_kernel.hpp"

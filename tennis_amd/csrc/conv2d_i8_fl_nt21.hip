// Flat-tile int8 convolution kernel, tiles of 2 + 1 position fragments.
#define TSX_FL_NTA 2
#define TSX_FL_NTB 1
#include "conv2d_i8_fl_kernel.hpp"

// Flat-tile int8 convolution kernel, tiles of 4 + 4 position fragments.
#define TSX_FL_NTA 4
#define TSX_FL_NTB 4
#include "conv2d_i8_fl_kernel.hpp"

// Flat-tile int8 convolution kernel, tiles of 2 + 2 position fragments.
#define TSX_FL_NTA 2
#define TSX_FL_NTB 2
#include "conv2d_i8_fl_kernel.hpp"

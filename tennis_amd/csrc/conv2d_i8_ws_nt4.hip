// Window-stationary int8 convolution kernel, tiles of 4 position fragments per wavefront.
#define TSX_WS_NT 4
#include "conv2d_i8_ws_kernel.hpp"

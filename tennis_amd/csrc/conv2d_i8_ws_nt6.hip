// Window-stationary int8 convolution kernel, tiles of 6 position fragments per wavefront.
#define TSX_WS_NT 6
#include "conv2d_i8_ws_kernel.hpp"

// Window-stationary int8 convolution kernel, tiles of 7 position fragments per wavefront.
#define TSX_WS_NT 7
#include "conv2d_i8_ws_kernel.hpp"

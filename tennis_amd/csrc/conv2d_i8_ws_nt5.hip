// Window-stationary int8 convolution kernel, tiles of 5 position fragments per wavefront.
#define TSX_WS_NT 5
#include "conv2d_i8_ws_kernel.hpp"

// Window-stationary int8 convolution kernel, tiles of 1 position fragment per wavefront.
#define TSX_WS_NT 1
#include "conv2d_i8_ws_kernel.hpp"

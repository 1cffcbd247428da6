// Chooses the TenniS API the "hip" backend is compiled against: the real TenniS headers
// (integration build, -DTSX_WITH_TENNIS with the TenniS include/ and src/ directories on the
// include path) or this repository's self-contained restatement of the same interfaces.
// A translation unit defines TSX_TS_QUANTIZED_OPS, TSX_TS_FLOAT_OPS or TSX_TS_GLUE_OPS before including this to
// get the operator skeletons it derives from (TenniS's two conv2d core headers clash).
#pragma once
#ifdef TSX_WITH_TENNIS
#ifdef TSX_TS_QUANTIZED_OPS
#include <backend/base/base_conv2d_quantized.h>
#include <backend/base/base_quantize.h>
#endif
#ifdef TSX_TS_FLOAT_OPS
#include <backend/base/base_batch_norm.h>
#include <backend/base/base_batch_scale.h>
#include <backend/base/base_fused_batch_norm.h>
#include <backend/base/base_add_bias.h>
#include <backend/base/base_activation.h>
#include <backend/base/base_conv2d.h>
#include <backend/base/base_conv2d_winograd.h>
#include <backend/base/base_inner_prod.h>
#include <backend/base/base_leaky_relu.h>
#endif
#ifdef TSX_TS_GLUE_OPS
#include <backend/base/base_add.h>
#include <backend/base/base_mul.h>
#include <backend/base/base_activation.h>
#include <backend/base/base_concat.h>
#include <backend/base/base_resize2d.h>
#include <backend/base/base_depthwise_conv2d.h>
#include <backend/base/base_global_pooling2d.h>
#include <backend/base/base_pooling2d.h>
#endif
#include <backend/base/operator_on_device.h>
#include <backend/name.h>
#include <core/device_context.h>
#include <core/tensor_builder.h>
#include <global/hard_allocator.h>
#include <global/hard_converter.h>
#include <global/memory_device.h>
#include <global/device_admin.h>
#include <global/operator_factory.h>
#include <runtime/stack.h>
#include <utils/ctxmgr_lite.h>
#include <utils/log.h>
#else
#include "../ts/base_ops.h"
#include "../ts/ts_api.h"
#endif

// Stand-in for OpenVINO's header of the same path: the rt_info keys of an execution graph.
#pragma once
#include "../standin.hpp"

namespace ov {
namespace exec_model_info {
static const char ORIGINAL_NAMES[] = "originalLayersNames";
static const char IMPL_TYPE[] = "primitiveType";
static const char OUTPUT_PRECISIONS[] = "outputPrecisions";
static const char PERF_COUNTER[] = "execTimeMcs";
static const char LAYER_TYPE[] = "layerType";
static const char EXECUTION_ORDER[] = "execOrder";
static const char RUNTIME_PRECISION[] = "runtimePrecision";
}  // namespace exec_model_info
}  // namespace ov

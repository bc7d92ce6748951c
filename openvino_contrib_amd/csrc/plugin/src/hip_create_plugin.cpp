// The symbol ov::Core resolves when it loads the plugin library: create_plugin_engine(), which
// hands back the Plugin object (modules/nvidia_plugin/src/cuda_create_plugin.cpp:11-12).
#include "hip_plugin.hpp"

#ifndef CI_BUILD_NUMBER
#define CI_BUILD_NUMBER "custom_hip_plugin"
#endif

namespace ov {
namespace hip_gpu {
namespace {

static const ov::Version version = {CI_BUILD_NUMBER, "openvino_hip_gpu_plugin"};
OV_DEFINE_PLUGIN_CREATE_FUNCTION(Plugin, version)

}  // namespace
}  // namespace hip_gpu
}  // namespace ov

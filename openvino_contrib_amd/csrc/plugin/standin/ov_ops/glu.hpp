// Stand-in for OpenVINO's header of the same path: everything is declared in openvino/standin.hpp.
#pragma once
#include "../openvino/standin.hpp"

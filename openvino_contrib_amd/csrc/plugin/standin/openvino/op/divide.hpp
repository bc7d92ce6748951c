// Stand-in for OpenVINO's header of the same path: everything is declared in standin.hpp.
#pragma once
#include "../standin.hpp"

// Stand-in for the NNabla core header of the same name; see core_min.hpp.
#pragma once
#include <nbla/core_min.hpp>

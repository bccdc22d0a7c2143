#pragma once
#include "ngraph/runtime/tensor.hpp"

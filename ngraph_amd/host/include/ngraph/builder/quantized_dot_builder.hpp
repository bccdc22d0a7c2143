// nGraph source path kept for unchanged #include lines; everything lives in ngraph/builder.hpp
#pragma once
#include "ngraph/builder.hpp"

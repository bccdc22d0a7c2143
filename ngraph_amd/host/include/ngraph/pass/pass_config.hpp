// nGraph source path kept for unchanged #include lines; everything lives in ngraph/pass.hpp
#pragma once
#include "ngraph/pass.hpp"

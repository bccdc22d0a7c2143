// path of the reference tree (src/ngraph/pass/pass.hpp); the classes live in ngraph/pass.hpp here
#pragma once
#include "ngraph/pass.hpp"

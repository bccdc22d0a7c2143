// Umbrella header, as src/ngraph/ngraph.hpp of the nGraph tree.
#pragma once
#include "ngraph/builder.hpp"
#include "ngraph/core.hpp"
#include "ngraph/ops.hpp"
#include "ngraph/pass.hpp"
#include "ngraph/runtime/backend.hpp"
#include "ngraph/runtime/backend_manager.hpp"
#include "ngraph/runtime/executable.hpp"
#include "ngraph/runtime/tensor.hpp"

// custos element-wise path for MI355X: expression DSL, module stack, HIP device.
#pragma once

#include "buffer.hpp"
#include "combiner.hpp"
#include "core.hpp"
#include "device.hpp"
#include "hip.hpp"
#include "modules.hpp"
#include "opt_graph.hpp"
#include "serde.hpp"

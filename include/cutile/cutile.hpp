// Umbrella header of the C++ host surface (the reference's `cutile::prelude`).
#pragma once
#include "api.hpp"
#include "bench.hpp"
#include "device_op.hpp"
#include "error.hpp"
#include "future.hpp"
#include "graph.hpp"
#include "runtime.hpp"
#include "tensor.hpp"
#include "tune.hpp"

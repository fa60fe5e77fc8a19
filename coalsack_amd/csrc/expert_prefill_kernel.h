// Expert MLP for the compute-bound (prefill) regime: grouped GEMM over the
// dispatched tokens.  (Filled in below.)
#pragma once
#include "common.h"
namespace csk {}

// Header name of the reference (include/pto/npu/a5/TMov.hpp): kernel sources that include the per-instruction headers of
// the NPU implementation get the instruction set of this library instead.
#pragma once
#include "pto/pto-inst.hpp"

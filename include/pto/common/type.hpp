// Element types and the instruction enumerations under the header name of the reference
// (include/pto/common/type.hpp:96-269).
#pragma once
#include "pto/common/types.hpp"

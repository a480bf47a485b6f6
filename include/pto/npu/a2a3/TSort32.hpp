// Header name of the reference, kept so that sources which include it compile: TSORT32 (include/pto/gfx950/sort_ops.hpp) come with <pto/pto-inst.hpp>.
#pragma once
#include <pto/pto-inst.hpp>

// Header name of the reference, kept so that sources which include it compile: the FIFO types of TPUSH / TPOP (DataFIFO, TPipe: include/pto/gfx950/fifo_ops.hpp) come with <pto/pto-inst.hpp>.
#pragma once
#include <pto/pto-inst.hpp>

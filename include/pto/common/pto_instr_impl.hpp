// Header name of the reference, kept so that sources which include it compile: the instruction implementations come with <pto/pto-inst.hpp>.
#pragma once
#include <pto/pto-inst.hpp>

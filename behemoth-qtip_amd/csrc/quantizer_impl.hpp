// group quantizer internals (filled in by quantizer_impl.cpp)
#pragma once
#include "qtip_internal.hpp"

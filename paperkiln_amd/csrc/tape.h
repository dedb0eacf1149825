// The autograd tape, device-resident: declared in include/paperkiln_amd.hpp (it is part of the
// library's C++ interface); this header adds the kernel launchers for the translation units that
// implement it.
#pragma once
#include "tensor.h"

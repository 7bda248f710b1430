// Host-side helpers shared by the C-ABI entry points.
#pragma once

#include <stdint.h>

namespace tk {

inline bool aligned_to(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

}  // namespace tk

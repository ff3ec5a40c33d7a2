// Test infrastructure: exposes the two helpers that RepDL declares in
// backend/cpu/math.h:14-15 (exp2d, log1d) but never binds to Python
// (backend/cpu/bind.cpp:12-18 has no bind_math).  Linked with the reference's own
// math.cpp object; contains no arithmetic of its own.
#include <torch/extension.h>

#include "math.h"

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("exp2d", &repdl::cpu::math::exp2d);
    m.def("log1d", &repdl::cpu::math::log1d);
}

// Module entry of the workspace extension. Fixed file: operators are added by dropping a
// kernels/<op>.hip + kernels/<op>_binding.cpp pair into the workspace, never by editing
// this file (agent_workdir/binding.cpp:4-9).
#include <pybind11/pybind11.h>

#include "binding_registry.h"

PYBIND11_MODULE(cuda_extension, m) {
    m.doc() = "gfx950 HIP operators of this workspace";
    BindingRegistry::getInstance().applyBindings(m);
    m.def("registered_bindings", []() { return BindingRegistry::getInstance().names(); },
          "names passed to REGISTER_BINDING, in registration order");
}

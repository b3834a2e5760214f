#pragma once
// Self-registration table for the operators of one workspace extension.
//
// Each kernels/<op>_binding.cpp places one REGISTER_BINDING(<op>, register_<op>) at file
// scope; the registrar object it defines runs while the shared object is being loaded, so
// by the time PyInit_cuda_extension calls applyBindings() every operator is in the table.
// Same classes, macro and behaviour as the reference workspace
// (agent_workdir/binding_registry.h:15-49): append-only, no duplicate check, applied in
// static-initialisation order, not thread-safe (loading is single-threaded).
//
// Only pybind11 is included here, never torch/extension.h, so that binding.cpp compiles in
// about a second.

#include <functional>
#include <string>
#include <utility>
#include <vector>

#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

class BindingRegistry {
public:
    using BindingFunction = std::function<void(pybind11::module&)>;

    BindingRegistry(const BindingRegistry&) = delete;
    BindingRegistry& operator=(const BindingRegistry&) = delete;

    // Function-local static: constructed on first use, which may be during another
    // translation unit's static initialisation.
    static BindingRegistry& getInstance() {
        static BindingRegistry the_registry;
        return the_registry;
    }

    void registerBinding(const std::string& name, BindingFunction func) {
        entries_.emplace_back(name, std::move(func));
    }

    void applyBindings(pybind11::module& m) {
        for (auto& entry : entries_) {
            entry.second(m);
        }
    }

    // Names in registration order (used by tests and error messages).
    std::vector<std::string> names() const {
        std::vector<std::string> out;
        out.reserve(entries_.size());
        for (const auto& entry : entries_) out.push_back(entry.first);
        return out;
    }

private:
    BindingRegistry() = default;
    std::vector<std::pair<std::string, BindingFunction>> entries_;
};

class BindingRegistrar {
public:
    BindingRegistrar(const std::string& name, BindingRegistry::BindingFunction func) {
        BindingRegistry::getInstance().registerBinding(name, std::move(func));
    }
};

#define REGISTER_BINDING(name, func) \
    static BindingRegistrar _registrar_##name(#name, [](pybind11::module& m) { func(m); })

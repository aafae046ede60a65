// PyGeNN extension module for the MI355X backend: `pygenn.mi355x_backend`, exporting what GeNNModel looks up in
// every backend module (pygenn/genn_model.py:108-140, 673-681): Preferences (every member settable the way
// `GeNNModel(..., backend="mi355x", kernel_source=..., step_queue_length=...)` sets them: keyword -> attribute),
// _Backend, _Runtime (the backend state of a loaded model) and _create_backend.  Built inside a PyGeNN source tree next
// to pygenn/src/hipBackend.cc (setup.py backend tuple ("mi355x", "mi355x", {...})); the only other change PyGeNN needs
// is "mi355x" in its list of backend names.  Mirrors pygenn/src/hipBackend.cc:28-86.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <plog/Appenders/ConsoleAppender.h>

#include "modelSpecInternal.h"

#include "optimiser.h"

using namespace GeNN;
using namespace GeNN::CodeGenerator::MI355X;

namespace
{
Backend makeBackend(const ModelSpecInternal &model, const std::string &outputPath,
                    plog::Severity backendLevel, const Preferences &preferences)
{
    // the appender has to outlive the logger it is handed to
    static plog::ConsoleAppender<plog::TxtFormatter> appender;
    return Optimiser::createBackend(model, filesystem::path(outputPath), backendLevel, &appender, preferences);
}
}

PYBIND11_MODULE(mi355x_backend, m)
{
    pybind11::module_::import("pygenn._genn");
    pybind11::module_::import("pygenn._runtime");

    pybind11::enum_<Preferences::KernelSource>(m, "KernelSource")
        .value("AUTO", Preferences::KernelSource::AUTO)
        .value("LIBRARY", Preferences::KernelSource::LIBRARY)
        .value("GENERATED", Preferences::KernelSource::GENERATED);

    pybind11::class_<Preferences, CodeGenerator::PreferencesBase>(m, "Preferences")
        .def(pybind11::init<>())
        .def_readwrite("device_id", &Preferences::deviceID)
        .def_readwrite("install_root", &Preferences::installRoot)
        .def_readwrite("kernel_source", &Preferences::kernelSource)
        .def_readwrite("ordered_accumulation", &Preferences::orderedAccumulation)
        .def_readwrite("step_queue_length", &Preferences::stepQueueLength)
        .def_readwrite("device_initialisation", &Preferences::deviceInitialisation)
        .def_readwrite("profiler_ranges", &Preferences::profilerRanges);

    pybind11::class_<State, Runtime::StateBase>(m, "_Runtime")
        .def_property_readonly("device_name", &State::getDeviceName)
        .def_property_readonly("free_device_mem_bytes", &State::getFreeDeviceMemBytes)
        .def("synchronize", &State::synchronize);

    pybind11::class_<Backend, CodeGenerator::BackendBase>(m, "_Backend")
        .def_property_readonly("kernels_generated", &Backend::areKernelsGenerated);

    m.def("_create_backend", &makeBackend, pybind11::return_value_policy::move);
}

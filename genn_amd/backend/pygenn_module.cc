// PyGeNN extension module for the MI355X backend: `pygenn.mi355x_backend`, exporting what GeNNModel looks up in
// every backend module (pygenn/genn_model.py:108-140): Preferences, _Backend and _create_backend.  Built inside a
// PyGeNN source tree next to pygenn/src/hipBackend.cc (setup.py backend tuple ("mi355x", "mi355x", {...})); the only
// other change PyGeNN needs is "mi355x" in its list of backend names.
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

    pybind11::class_<Preferences, CodeGenerator::PreferencesBase>(m, "Preferences")
        .def(pybind11::init<>())
        .def_readwrite("device_id", &Preferences::deviceID)
        .def_readwrite("install_root", &Preferences::installRoot);

    pybind11::class_<Backend, CodeGenerator::BackendBase>(m, "_Backend");

    m.def("_create_backend", &makeBackend, pybind11::return_value_policy::move);
}

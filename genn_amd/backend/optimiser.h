#pragma once
// Entry point GeNN's generator and PyGeNN look up in every backend
// (include/genn/backends/single_threaded_cpu/optimiser.h, src/genn/generator/generator.cc:28-30).
#include <plog/Severity.h>

#include "backendExport.h"
#include "backend.h"

namespace GeNN { class ModelSpecInternal; }
namespace plog { class IAppender; }

namespace GeNN::CodeGenerator::MI355X::Optimiser
{
BACKEND_EXPORT Backend createBackend(const ModelSpecInternal &model, const filesystem::path &outputPath,
                                     plog::Severity backendLevel, plog::IAppender *backendAppender,
                                     const Preferences &preferences);
}

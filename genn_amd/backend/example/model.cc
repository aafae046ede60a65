// A model file for genn-buildmodel (the reference's C++ front end: bin/genn-buildmodel.sh builds src/genn/generator/generator.cc
// with -DMODEL="<this file>" and -DBACKEND_NAMESPACE=<backend>, generator.cc:28-121): the balanced network of 3,200
// excitatory and 800 inhibitory LIF neurons (Vogels-Abbott shape, the first benchmark configuration) written against
// GeNN's own ModelSpec API with nothing but built-in snippets, so that the same file runs on the reference's
// SingleThreadedCPU backend and on the MI355X backend.  Connectivity and initial potentials come from GeNN's seeded
// initialisation snippets; both backends run that initialisation on the host with the same generator, so the two runs
// must produce the same spikes.
#include <cstdlib>
#include <iostream>

#include "modelSpec.h"

void modelDefinition(ModelSpec &model)
{
    model.setDT(0.1);
    model.setName("balanced");
    model.setSeed(1234);
    model.setPrecision(Type::Float);

    const ParamValues lif{{"C", 1.0}, {"TauM", 20.0}, {"Vrest", -60.0}, {"Vreset", -60.0}, {"Vthresh", -50.0}, {"Ioffset", 0.55}, {"TauRefrac", 5.0}};
    const VarValues state{{"V", initVar<InitVarSnippet::Uniform>({{"min", -60.0}, {"max", -50.0}})}, {"RefracTime", 0.0}};
    auto *e = model.addNeuronPopulation<NeuronModels::LIF>("E", 3200, lif, state);
    auto *i = model.addNeuronPopulation<NeuronModels::LIF>("I", 800, lif, state);
    e->setSpikeRecordingEnabled(true);
    i->setSpikeRecordingEnabled(true);

    const auto connect = [](){ return initConnectivity<InitSparseConnectivitySnippet::FixedProbability>({{"prob", 0.02}}); };
    const auto excitatory = [](){ return initWeightUpdate<WeightUpdateModels::StaticPulseConstantWeight>({{"g", 0.5}}); };
    const auto inhibitory = [](){ return initWeightUpdate<WeightUpdateModels::StaticPulseConstantWeight>({{"g", -2.25}}); };
    const auto fast = [](){ return initPostsynaptic<PostsynapticModels::ExpCurr>({{"tau", 5.0}}); };
    const auto slow = [](){ return initPostsynaptic<PostsynapticModels::ExpCurr>({{"tau", 10.0}}); };
    model.addSynapsePopulation("EE", SynapseMatrixType::SPARSE, e, e, excitatory(), fast(), connect());
    model.addSynapsePopulation("EI", SynapseMatrixType::SPARSE, e, i, excitatory(), fast(), connect());
    model.addSynapsePopulation("IE", SynapseMatrixType::SPARSE, i, e, inhibitory(), slow(), connect());
    model.addSynapsePopulation("II", SynapseMatrixType::SPARSE, i, i, inhibitory(), slow(), connect());
}

// generator.cc:119-121 hands the built model to this function.  GENN_EXAMPLE_STEPS (default 0: build only) timesteps
// are simulated; per population the number of spikes and an order-sensitive checksum of the (step, neuron) raster are printed.
void simulate(ModelSpec &model, Runtime::Runtime &runtime)
{
    const char *env = std::getenv("GENN_EXAMPLE_STEPS");
    const unsigned long steps = env ? std::strtoul(env, nullptr, 10) : 0ul;
    if(steps == 0) {
        std::cout << "example: built " << model.getName() << " (set GENN_EXAMPLE_STEPS to simulate)" << std::endl;
        return;
    }
    runtime.allocate(steps);
    runtime.initialize();
    runtime.initializeSparse();
    for(unsigned long s = 0; s < steps; s++) { runtime.stepTime(); }
    runtime.pullRecordingBuffersFromDevice();
    for(const char *name : {"E", "I"}) {
        const auto events = runtime.getRecordedSpikes(*model.findNeuronGroup(name));
        const auto &times = events.at(0).first;
        const auto &ids = events.at(0).second;
        // spikes of one timestep are listed in bit-scan order of the recording words, the same on every backend
        unsigned long long checksum = 1469598103934665603ull;
        for(size_t k = 0; k < ids.size(); k++) {
            const unsigned long long step = (unsigned long long)(times[k] / 0.1 + 0.5);
            checksum = (checksum ^ (step * 1000003ull + ids[k])) * 1099511628211ull;
        }
        std::cout << "example: population " << name << " spikes " << ids.size() << " checksum " << checksum << std::endl;
    }
}

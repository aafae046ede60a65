"""The selection boundary: the reference selects a backend at compile time — bin/genn-buildmodel.sh builds
src/genn/generator/generator.cc with -DMODEL="<model file>" and -DBACKEND_NAMESPACE=<namespace> plus the include path of the
backend's optimiser.h (src/genn/generator/MakefileCommon, generator.cc:28-121) — and PyGeNN by importing
pygenn.<name>_backend (pygenn/genn_model.py:106-120).  oracle/Makefile.ref compiles the reference's generator.cc where it
lies with the name and namespace read from genn_amd/backend/MakefileMI355X and the example model file
genn_amd/backend/example/model.cc; these tests run the result (no GPU needed: the example simulates nothing unless asked) and
apply the patch that lists the backend in the GeNN tree."""
import ast
import json
import os
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GENERATOR = os.path.join(ROOT, "oracle", "_ref", "mi355x_generator")
REFERENCE = "/root/reference"
BACKEND_DIR = os.path.join(ROOT, "genn_amd", "backend")


def _exports(lib):
    out = subprocess.run(["nm", "-D", "--defined-only", lib], stdout=subprocess.PIPE, text=True, check=True).stdout
    return {line.split()[-1] for line in out.splitlines() if " T " in line or " B " in line or " D " in line}


def test_generator_configuration_names_the_backend():
    text = open(os.path.join(BACKEND_DIR, "MakefileMI355X")).read()
    assert "BACKEND_NAME        :=mi355x" in text and "BACKEND_NAMESPACE   :=MI355X" in text and "include MakefileCommon" in text
    # the namespace the generator is compiled with must be the one backend.h declares
    assert "namespace GeNN::CodeGenerator::MI355X" in open(os.path.join(BACKEND_DIR, "backend.h")).read()
    assert "mi355x_backend" in open(os.path.join(BACKEND_DIR, "pygenn_module.cc")).read()


def test_pygenn_module_exposes_every_preference_and_the_backend_state():
    """PyGeNN sets backend preferences by attribute (pygenn/genn_model.py:673-681: every keyword of GeNNModel that is not a
    model option becomes `setattr(preferences, name, value)`), so every member of the backend's Preferences struct must be
    bound, under its snake_case name, and the backend state must be there under the name PyGeNN looks up (`_Runtime`,
    pygenn/src/hipBackend.cc:57-67).  `pygenn._genn` is not built here, so the module cannot be imported: the check is
    of the source against the struct, plus the module having been compiled (its init symbol)."""
    import re
    header = open(os.path.join(BACKEND_DIR, "backend.h")).read()
    struct = header[header.index("struct Preferences"):header.index("void updateHash")]
    members = re.findall(r"^\s+(?:int|bool|unsigned int|std::string|KernelSource)\s+(\w+)\s*(?:=[^;]*)?;", struct, flags=re.M)
    assert set(members) == {"deviceID", "installRoot", "kernelSource", "orderedAccumulation", "stepQueueLength", "deviceInitialisation", "profilerRanges"}, members
    module = open(os.path.join(BACKEND_DIR, "pygenn_module.cc")).read()
    for member in members:
        snake = re.sub(r"(?<=[a-z])([A-Z])", lambda m: "_" + m.group(1).lower(), member).replace("_i_d", "_id").lower()
        assert f'.def_readwrite("{snake}", &Preferences::{member})' in module, (member, snake)
    for value in ("AUTO", "LIBRARY", "GENERATED"):
        assert f'.value("{value}", Preferences::KernelSource::{value})' in module
    assert 'pybind11::class_<State, Runtime::StateBase>(m, "_Runtime")' in module
    assert '"_Backend"' in module and '"_create_backend"' in module
    import sysconfig
    built = os.path.join(ROOT, "genn_amd", "lib", "mi355x_backend" + sysconfig.get_config_var("EXT_SUFFIX"))
    if os.path.exists(built):
        assert "PyInit_mi355x_backend" in _exports(built)


@pytest.mark.skipif(not os.path.exists(GENERATOR), reason="oracle/_ref/mi355x_generator is not built (needs the reference tree at build time)")
def test_reference_generator_selects_the_backend_and_builds_a_runner():
    """generator.cc as genn-buildmodel runs it: <genn dir> <target dir> <force rebuild>.  It creates the backend through
    Optimiser::createBackend of the selected namespace, generates and compiles <model>_CODE/librunner.so and hands model and
    Runtime to the model file's simulate(), which only reports when GENN_EXAMPLE_STEPS is unset."""
    tmp = tempfile.mkdtemp(prefix="selection_")
    try:
        env = dict(os.environ)
        env.pop("GENN_EXAMPLE_STEPS", None)
        res = subprocess.run([GENERATOR, REFERENCE, tmp, "1"], cwd=tmp, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert res.returncode == 0, res.stdout[-3000:]
        assert "example: built balanced" in res.stdout
        code = os.path.join(tmp, "balanced_CODE")
        exports = _exports(os.path.join(code, "librunner.so"))
        for name in ("allocateMem", "freeMem", "initialize", "initializeSparse", "initializeHost", "stepTime", "updateNeurons", "updateSynapses",
                     "neuronUpdateTime", "presynapticUpdateTime", "postsynapticUpdateTime", "initTime", "initSparseTime"):
            assert name in exports, f"{name} missing from the generated runner"
        assert any(e.startswith("pushMergedNeuronUpdateGroup") for e in exports) and any(e.startswith("pushMergedPresynapticUpdateGroup") for e in exports)
        ldd = subprocess.run(["ldd", os.path.join(code, "librunner.so")], stdout=subprocess.PIPE, text=True).stdout
        assert "libgenn_mi355x.so" in ldd
        # the built-in initialisation snippets the model uses run through the reference's host-side init code
        init = open(os.path.join(code, "init.cc")).read()
        assert "gennmi_push_mirrors" in init
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_golden_of_the_example_model_is_from_the_reference_backend():
    golden = json.load(open(os.path.join(ROOT, "tests", "golden", "selection_example.json")))
    assert golden["steps"] == 3000 and set(golden["populations"]) == {"E", "I"}
    assert all(p["spikes"] > 1000 for p in golden["populations"].values())


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "pygenn")), reason="needs the reference tree")
def test_tree_patch_applies_to_the_reference():
    """genn_tree.patch lists the backend where the GeNN tree lists its backends: the import loop of pygenn/genn_model.py, the
    getopts of bin/genn-buildmodel.sh, the backend tuples of setup.py and the backend targets of the top-level Makefile."""
    tmp = tempfile.mkdtemp(prefix="tree_patch_")
    try:
        files = ("pygenn/genn_model.py", "bin/genn-buildmodel.sh", "setup.py", "Makefile")
        for f in files:
            os.makedirs(os.path.dirname(os.path.join(tmp, f)), exist_ok=True)
            shutil.copy(os.path.join(REFERENCE, f), os.path.join(tmp, f))
        with open(os.path.join(BACKEND_DIR, "genn_tree.patch")) as patch:
            res = subprocess.run(["patch", "-p1", "--no-backup-if-mismatch"], cwd=tmp, stdin=patch, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        assert res.returncode == 0, res.stdout
        assert 'for b in ["mi355x", "cuda", "hip", "single_threaded_cpu"]' in open(os.path.join(tmp, files[0])).read()
        script = open(os.path.join(tmp, files[1])).read()
        assert 'x) GENERATOR_MAKEFILE="MakefileMI355X";;' in script and 'getopts "clpxdvfs:o:i:h"' in script
        assert subprocess.run(["bash", "-n", os.path.join(tmp, files[1])]).returncode == 0
        setup = open(os.path.join(tmp, files[2])).read()
        ast.parse(setup)
        ast.parse(open(os.path.join(tmp, files[0])).read())
        assert 'backends.append(("mi355x", "mi355x"' in setup
        makefile = open(os.path.join(tmp, files[3])).read()
        assert "mi355x_backend: genn" in makefile and "$(MAKE) -C src/genn/backends/mi355x" in makefile
    finally:
        shutil.rmtree(tmp, ignore_errors=True)

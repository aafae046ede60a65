"""Writes tests/golden/selection_example.json: spike counts and raster checksums of genn_amd/backend/example/model.cc
run by the reference's OWN generator driver (src/genn/generator/generator.cc) on the reference's SingleThreadedCPU
backend — oracle/_ref/ref_generator, built by oracle/Makefile.ref in the builder container.  The GPU test runs the same
model file through the same driver built with -DBACKEND_NAMESPACE=MI355X and must print the same lines."""
import json
import os
import re
import subprocess
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
STEPS = 3000


def main():
    gen = os.path.join(ROOT, "oracle", "_ref", "ref_generator")
    with tempfile.TemporaryDirectory(prefix="selection_golden_") as tmp:
        res = subprocess.run([gen, "/root/reference", tmp, "1"], cwd=tmp, env=dict(os.environ, GENN_EXAMPLE_STEPS=str(STEPS)),
                             stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, check=True)
    pops = {m.group(1): {"spikes": int(m.group(2)), "checksum": m.group(3)}
            for m in re.finditer(r"example: population (\w+) spikes (\d+) checksum (\d+)", res.stdout)}
    assert set(pops) == {"E", "I"}, res.stdout[-2000:]
    with open(os.path.join(ROOT, "tests", "golden", "selection_example.json"), "w") as f:
        json.dump({"steps": STEPS, "populations": pops}, f, indent=1, sort_keys=True)
        f.write("\n")
    print(pops)


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Writes the golden fixtures tests/golden/<case>.npz by running the REFERENCE's own
SingleThreadedCPU backend (oracle/_ref/ref_driver, built by oracle/Makefile.ref from the sources
under /root/reference) on each case of cases.py.  Runs only where the reference tree is mounted;
the fixtures it writes are data: the digest of the inputs, spike rasters, and state snapshots.

    python tests/golden/make_golden.py [case ...]
"""
import os
import shutil
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

from genn_amd.netspec import write_netspec  # noqa: E402
from cases import CASES  # noqa: E402

DRIVER = os.path.join(ROOT, "oracle", "_ref", "ref_driver")


def make(name):
    net, snap = CASES[name]()
    net.snap = snap
    tmp = tempfile.mkdtemp(prefix="golden_")
    try:
        spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
        for d in (work, out):
            os.makedirs(d)
        write_netspec(net, spec)
        subprocess.check_call([DRIVER, spec, work, out], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        data = {"input_digest": np.array(net.input_digest()), "snap": np.array(snap), "steps": np.array(net.steps)}
        fuse = dict(line.split() for line in open(os.path.join(out, "fusemap.txt")))
        data["fusemap"] = np.array([f"{k}={v}" for k, v in fuse.items()])
        for p in net.pops:
            data[f"spikes.{p.name}"] = np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32).reshape(-1, 2)
            for var in ("V", "RefracTime", "U", "A"):
                f = os.path.join(out, f"{p.name}.{var}.f32")
                if os.path.exists(f):
                    data[f"{var}.{p.name}"] = np.fromfile(f, np.float32).reshape(-1, p.n)
        for s in net.syns:
            for var, dtype in (("outPost", np.float32), ("denDelay", np.float32), ("g", np.float32), ("preTrace", np.float32),
                               ("postTrace", np.float32), ("colLength", np.uint32), ("remap", np.uint32),
                               ("wPre", np.float32), ("wPost", np.float32), ("sPre", np.float32), ("sPost", np.float32), ("x", np.float32), ("hits", np.float32)):
                f = os.path.join(out, f"{s.name}.{var}.{'u32' if dtype == np.uint32 else 'f32'}")
                if os.path.exists(f):
                    a = np.fromfile(f, dtype)
                    if var in ("g", "denDelay", "outPost", "preTrace", "postTrace", "wPre", "wPost", "sPre", "sPost", "x", "hits"):
                        a = a.reshape(net.steps // snap, -1)[-1] if var in ("g", "denDelay") else a.reshape(net.steps // snap, -1)
                    data[f"{var}.{s.name}"] = a
            f = os.path.join(out, f"{s.name}.events.u32")
            if os.path.exists(f):
                data[f"events.{s.name}"] = np.fromfile(f, np.uint32).reshape(-1, 2)
            f = os.path.join(out, f"{s.name}.colStride.txt")
            if os.path.exists(f):
                data[f"colStride.{s.name}"] = np.array(int(open(f).read()))
        # variables of custom updates and what they wrote into the projections they refer to: one row per snapshot
        for c in net.customs:
            for var in ("applied", "sum", "peak", "total", "when", "w", "transposed", "removed", "born"):
                f = os.path.join(out, f"{c.name}.{var}.f32")
                if os.path.exists(f):
                    data[f"custom.{c.name}.{var}"] = np.fromfile(f, np.float32).reshape(net.steps // snap, -1)
            for var in ("rowLength", "ind", "next"):
                f = os.path.join(out, f"{c.name}.{var}.u32")
                if os.path.exists(f):
                    data[f"custom.{c.name}.{var}"] = np.fromfile(f, np.uint32).reshape(net.steps // snap, -1)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)
        total = sum(len(data[f"spikes.{p.name}"]) for p in net.pops)
        print(f"{name}: {total} spikes, {os.path.getsize(os.path.join(HERE, name + '.npz')) / 1024:.0f} KiB")
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def make_poisson_rates():
    """potjans_poisson_rates.npz: spike counts per population of the scaled cortical microcircuit under its PoissonExp
    background, run by the reference's CPU backend for 5 s of model time under two seeds.  The reference draws the
    background from its host generator, which no other backend reproduces, so what these runs fix is the statistics:
    the mean rates, and (from the two seeds) how far two correct runs differ."""
    from cases import potjans_poisson_net
    data = {}
    for seed in (1234, 98765):
        net = potjans_poisson_net()
        net.seed = seed
        net.snap = net.steps
        tmp = tempfile.mkdtemp(prefix="golden_")
        try:
            spec, work, out = (os.path.join(tmp, d) for d in ("spec", "work", "out"))
            for d in (work, out):
                os.makedirs(d)
            write_netspec(net, spec)
            subprocess.check_call([DRIVER, spec, work, out], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
            counts = [len(np.fromfile(os.path.join(out, f"{p.name}.spikes.u32"), np.uint32)) // 2 for p in net.pops]
            data[f"counts.{seed}"] = np.array(counts, np.int64)
            print(seed, {p.name: round(c / p.n / (net.steps * net.dt / 1000.0), 3) for p, c in zip(net.pops, counts)})
        finally:
            shutil.rmtree(tmp, ignore_errors=True)
    data["input_digest"] = np.array(net.input_digest())
    data["steps"] = np.array(net.steps)
    data["sizes"] = np.array([p.n for p in net.pops], np.int64)
    np.savez_compressed(os.path.join(HERE, "potjans_poisson_rates.npz"), **data)


if __name__ == "__main__":
    if not os.path.exists(DRIVER):
        raise SystemExit("oracle/_ref/ref_driver is missing: run `make -f Makefile.ref` in oracle/ (needs /root/reference)")
    for case in (sys.argv[1:] or list(CASES) + ["potjans_poisson_rates"]):
        make_poisson_rates() if case == "potjans_poisson_rates" else make(case)

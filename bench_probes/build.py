"""Compile the two measurement aids of bench.py (a matrix-core-only loop and a read-only
launch) into bench_probes/libk3q_probe.so for gfx950.  Not part of the product library: the
package never loads it.  Run as `python -m bench_probes.build` or through
`__graft_entry__.build()`."""

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libk3q_probe.so")
SOURCES = ["probe_mfma.hip", "probe_stream.hip"]


def build(verbose=True):
    from keras_amd.csrc.build import FLAGS, hipcc

    cmd = [hipcc(), *FLAGS, "-shared", "-o", LIB, *[os.path.join(HERE, s) for s in SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if out.returncode != 0:
        sys.stderr.write(out.stdout.decode())
        raise RuntimeError("hipcc failed on the probe library")
    return LIB


if __name__ == "__main__":
    sys.path.insert(0, os.path.dirname(HERE))
    build()

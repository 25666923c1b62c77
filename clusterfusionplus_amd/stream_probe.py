"""Builds and runs the bare read probes of csrc/stream_probe.hip (streaming rate and dependent round-trip latency by
waves per compute unit and loads in flight; warm against cold reads).  A measurement tool: nothing in the library uses it.

    python -m clusterfusionplus_amd.build --stream-probe     # on the build machine (hipcc cross-compiles for gfx950)
    python clusterfusionplus_amd/stream_probe.py             # on the MI355X; prints the table profiles/stream_ceiling.txt holds
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "stream_probe_bin")


def main():
    if not os.path.exists(BIN):
        print(f"{BIN} is not built: run `python -m clusterfusionplus_amd.build --stream-probe` first", file=sys.stderr)
        return 2
    return subprocess.run([BIN]).returncode


if __name__ == "__main__":
    sys.exit(main())

"""Compile the table of an irreps triple into the library.

    python -m equitorch_amd.csrc.register NAME IRREPS_OUT IRREPS_IN1 IRREPS_IN2

adds ``NAME: [IRREPS_OUT, IRREPS_IN1, IRREPS_IN2]`` to ``extra_uvu_configs.json`` next to this file and rebuilds
``libcgtp.so``; from then on channel-wise products of these irreps (row mode and the fused edge path) run on
straight-line code generated for their table, like the irreps compiled in by default, instead of on the table-driven
kernels.  ``NAME`` must be a C identifier.  Without arguments: lists what is registered.
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PATH = os.path.join(HERE, "extra_uvu_configs.json")


def main(argv) -> int:
    registered = {}
    if os.path.exists(PATH):
        with open(PATH) as f:
            registered = json.load(f)
    if not argv:
        for name, triple in registered.items():
            print(name, *triple)
        return 0
    if len(argv) != 4 or not argv[0].isidentifier():
        print(__doc__, file=sys.stderr)
        return 2
    from ..irreps import Irreps
    name, triple = argv[0], list(argv[1:])
    for s in triple:
        Irreps(s)              # raises on a malformed string before anything is written
    registered[name] = triple
    with open(PATH, "w") as f:
        json.dump(registered, f, indent=1)
    from . import build
    print(build.build())
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))

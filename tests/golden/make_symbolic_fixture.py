#!/usr/bin/env python3
"""Writes tests/golden/reference_symbolics.json: the ``opmx::`` ONNX nodes (kind, input and
output counts, attribute names and values) that the REFERENCE's ``torch_function`` operators
emit for the calls listed in ``symbolic_cases.py``.

Run in the build container only, where the reference checkout is mounted:

    python tests/golden/make_symbolic_fixture.py /root/reference

The reference package is imported (its ``symbolic`` / export-placeholder branches run on small CPU
tensors; no eager operator arithmetic is involved); nothing of it is copied.  The fixture holds
data only and is what ``tests/test_host_wrappers.py`` compares this build's exports with."""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    sys.path.insert(0, ref)
    sys.path.insert(0, HERE)
    import torch
    import torch_function as OPMX          # the reference's package
    assert os.path.abspath(OPMX.__file__).startswith(os.path.abspath(ref)), OPMX.__file__
    from symbolic_cases import cases, export_nodes
    torch.manual_seed(0)
    out = {}
    for name, mod, args in cases(OPMX):
        out[name] = export_nodes(mod, args)
    with open(os.path.join(HERE, "reference_symbolics.json"), "w") as f:
        json.dump({"source": "OpenPPL/ppl.pmx torch_function symbolic() functions, torch {}".format(torch.__version__),
                   "nodes": out}, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", len(out), "cases")


if __name__ == "__main__":
    main()
